"""CPU tests: the oracle's integer planners pinned by brute force / closed forms / the reference's known
answers, and the product's host planners (C ABI, no GPU needed) checked bit-for-bit against the oracle."""

import logging

import numpy as np
import pytest
import torch

from oracle import sp_oracle, vit_oracle


def _ops():
    from mi355_vit import ops

    return ops


# ----------------------------------------------------------------------------------- brute-force models
def naive_window_index(grid, merge=2, window=112, patch=14):
    """2-D raster scan: visit windows (frame, wr, wc) in order and, inside each, units row-major."""
    win = window // merge // patch
    idx, cu, base = [], [0], 0
    for t, h, w in grid:
        gh, gw = h // merge, w // merge
        for f in range(t):
            for wr in range(0, gh, win):
                for wc in range(0, gw, win):
                    n = 0
                    for r in range(wr, min(wr + win, gh)):
                        for c in range(wc, min(wc + win, gw)):
                            idx.append(base + (f * gh + r) * gw + c)
                            n += 1
                    cu.append(cu[-1] + n * merge * merge)
        base += t * gh * gw
    return idx, cu


def naive_pos_ids(grid, merge=2):
    out = []
    for t, h, w in grid:
        frame = []
        for br in range(h // merge):
            for bc in range(w // merge):
                for dy in range(merge):
                    for dx in range(merge):
                        frame.append((br * merge + dy, bc * merge + dx))
        out += frame * t
    return out


GRIDS = [[(1, 16, 16)], [(1, 2, 2)], [(2, 6, 10)], [(1, 18, 22), (2, 8, 12), (1, 34, 16)], [(3, 8, 8), (1, 10, 26)]]


@pytest.mark.parametrize("grid", GRIDS)
def test_window_index_oracle_and_product_match_raster_scan(grid):
    idx_ref, cu_ref = naive_window_index(grid)
    idx_o, cu_raw = vit_oracle.window_index(grid, 2, 112, 14)
    assert idx_o.tolist() == idx_ref
    assert vit_oracle.dedup_cu(cu_raw).tolist() == cu_ref
    idx_p, cu_p = _ops().window_index(torch.tensor(grid), 2, 112, 14)
    assert idx_p.tolist() == idx_ref and cu_p.tolist() == cu_ref and cu_p.dtype == torch.int32
    # invariants: a permutation; strictly increasing boundaries ending at S
    S = sum(t * h * w for t, h, w in grid)
    assert sorted(idx_ref) == list(range(S // 4)) and cu_ref[-1] == S and all(b > a for a, b in zip(cu_ref, cu_ref[1:]))


def test_window_index_all_small_grids():
    ops = _ops()
    for gh in range(1, 13):
        for gw in range(1, 13):
            grid = [(1, 2 * gh, 2 * gw)]
            idx_ref, cu_ref = naive_window_index(grid)
            idx_o, cu_raw = vit_oracle.window_index(grid, 2, 112, 14)
            idx_p, cu_p = ops.window_index(torch.tensor(grid), 2, 112, 14)
            assert idx_o.tolist() == idx_ref == idx_p.tolist(), grid
            assert vit_oracle.dedup_cu(cu_raw).tolist() == cu_ref == cu_p.tolist(), grid


def test_window_index_hand_answers():
    idx, cu = vit_oracle.window_index([(1, 16, 16)], 2, 112, 14)
    # 8x8 merged units, 4x4-unit windows: the first window holds rows 0-3 x cols 0-3
    assert idx[:16].tolist() == [0, 1, 2, 3, 8, 9, 10, 11, 16, 17, 18, 19, 24, 25, 26, 27]
    assert vit_oracle.dedup_cu(cu).tolist() == [0, 64, 128, 192, 256]
    # the evenly-divisible case enumerates a band of empty windows: repeated entries before de-duplication
    assert len(cu) > 5 and len(set(cu)) == 5


@pytest.mark.parametrize("grid", GRIDS)
def test_rot_pos_ids(grid):
    ref = naive_pos_ids(grid)
    assert vit_oracle.rot_pos_ids(grid, 2).tolist() == [list(p) for p in ref]
    assert _ops().rot_pos_ids(torch.tensor(grid), 2).tolist() == [list(p) for p in ref]


def test_cu_seqlens_per_frame():
    grid = [(1, 16, 16), (8, 32, 56), (2, 4, 6)]
    want = [0, 256] + [256 + 1792 * (i + 1) for i in range(8)] + [256 + 8 * 1792 + 24, 256 + 8 * 1792 + 48]
    assert vit_oracle.cu_seqlens(grid).tolist() == want
    got = _ops().cu_seqlens(torch.tensor(grid))
    assert got.tolist() == want and got.dtype == torch.int32


def test_rotary_table_closed_form():
    grid = [(2, 4, 6)]
    inv = vit_oracle.default_inv_freq(80)
    assert inv.shape == (20,) and inv[0] == 1.0 and torch.isclose(inv[1], torch.tensor(10000.0 ** (-2 / 40)))
    tab = vit_oracle.rotary_table(grid, 2, inv)
    ids = naive_pos_ids(grid)
    for n in (0, 5, 17, 47):
        h, w = ids[n]
        assert torch.allclose(tab[n], torch.cat([h * inv, w * inv]))
    # bf16 buffers give a bf16 table (the reference's dtype propagation)
    assert vit_oracle.rotary_table(grid, 2, inv.to(torch.bfloat16)).dtype == torch.bfloat16


def test_planner_argument_errors():
    ops = _ops()
    with pytest.raises(RuntimeError, match="multiples of 2"):
        ops.window_index(torch.tensor([[1, 15, 16]]), 2, 112, 14)
    with pytest.raises(RuntimeError):
        ops.rot_pos_ids(torch.tensor([[0, 4, 4]]), 2)


# ----------------------------------------------------------------------------------- sequence-parallel cuts
def test_token_cuts_reference_known_answers():
    ops = _ops()
    for fn in (sp_oracle.token_cuts, ops.sp_token_cuts):
        assert np.diff(fn(8, 2)).tolist() == [4, 4] and np.diff(fn(12, 2)).tolist() == [6, 6]
        assert np.diff(fn(7, 3)).tolist() == [3, 2, 2] and np.diff(fn(11, 3)).tolist() == [4, 4, 3]
        assert np.diff(fn(100, 4)).tolist() == [25] * 4
        assert np.diff(fn(2, 4)).tolist() == [1, 1, 0, 0]


def test_window_cuts_reference_known_answers():
    ops = _ops()
    for fn in (sp_oracle.window_cuts, ops.sp_window_cuts):
        assert fn(10, 2, [6, 4])[0] == [0, 6, 10] and fn(14, 2, [7, 7])[0] == [0, 7, 14]
        pos, idx = fn(5, 4, [5])
        assert sorted(np.diff(pos).tolist()) == [0, 0, 0, 5] and idx[-1] == 1
    with pytest.raises(ValueError, match="no window lengths"):
        sp_oracle.window_cuts(5, 2, [])
    with pytest.raises(ValueError, match="no window lengths"):
        ops.sp_window_cuts(5, 2, [])
    with pytest.raises(ValueError, match="do not sum"):
        ops.sp_window_cuts(6, 2, [2, 3])
    with pytest.raises(ValueError, match="non-positive"):
        ops.sp_window_cuts(5, 2, [5, 0])


def test_window_cuts_brute_force_properties_and_product_equals_oracle():
    ops = _ops()
    rng = np.random.default_rng(0)
    for _ in range(300):
        nw = int(rng.integers(1, 12))
        wl = rng.integers(1, 65, nw).tolist()
        n = sum(wl)
        prefix = np.concatenate([[0], np.cumsum(wl)]).tolist()
        for sp in range(1, 9):
            pos, idx = sp_oracle.window_cuts(n, sp, wl)
            assert (pos, idx) == ops.sp_window_cuts(n, sp, wl)
            assert pos[0] == 0 and pos[-1] == n and len(pos) == sp + 1
            assert all(b >= a for a, b in zip(pos, pos[1:])) and all(p in prefix for p in pos)
            assert [prefix[i] for i in idx] == pos
            if nw >= sp:  # enough windows: every cut is the first boundary at or after k*n/sp unless clamped
                for k in range(1, sp):
                    want = next(p for p in prefix if p >= n * k // sp)
                    assert pos[k] <= max(want, pos[k - 1]) or idx[k] == len(prefix) - (sp - k)


def test_plan_split_matches_oracle_and_reference_answers(caplog):
    from mi355_vit import sequence_parallel_utils as spu

    m0 = spu.plan_split([8, 12], 0, 2)
    m1 = spu.plan_split([8, 12], 1, 2)
    assert m0.local_lengths == [4, 6] and m0.total_local_len == 10 and m1.local_lengths == [4, 6]
    assert m0.sample_global_slices == [(0, 4), (8, 14)] and m1.sample_global_slices == [(4, 8), (14, 20)]
    assert [spu.plan_split([7, 11], r, 3).local_lengths for r in range(3)] == [[3, 4], [2, 4], [2, 3]]
    m = spu.plan_split([2], 2, 4)
    assert m.total_local_len == 0 and m.requires_dummy_pad and m.batch_size == 1
    # windowed: global cu_window [0, 6, 10, 17, 24], samples [10, 14], rank 0 of 2 -> [0, 6, 13]
    cu = torch.tensor([0, 6, 10, 17, 24], dtype=torch.int32)
    mw = spu.plan_split([10, 14], 0, 2, cu_window_seqlens=cu)
    assert spu.rebuild_local_cu_seqlens(mw, use_windows=True).tolist() == [0, 6, 13]
    assert spu.rebuild_local_cu_seqlens(mw).dtype == torch.int32
    assert sp_oracle.local_window_cu(mw.window_lengths_per_sample, mw.window_index_ranges).tolist() == [0, 6, 13]
    # plain cu_seqlens
    plain = spu.plan_split([4, 7, 2], 0, 1)
    assert spu.rebuild_local_cu_seqlens(plain).tolist() == [0, 4, 11, 13] == sp_oracle.local_cu([4, 7, 2]).tolist()
    # fewer windows than ranks: one rank gets everything, a warning is logged on rank 0
    caplog.set_level(logging.WARNING)
    lens = [spu.plan_split([5], r, 4, cu_window_seqlens=torch.tensor([0, 5], dtype=torch.int32)).local_lengths[0] for r in range(4)]
    assert sorted(lens) == [0, 0, 0, 5] and "Sequence parallel requested" in caplog.text
    with pytest.raises(ValueError, match="Window metadata not available"):
        spu.rebuild_local_cu_seqlens(plain, use_windows=True)
    with pytest.raises(ValueError, match="do not cover sample"):
        spu.plan_split([10, 14], 0, 2, cu_window_seqlens=torch.tensor([0, 6, 11, 24], dtype=torch.int32))
    # random agreement with the oracle, all ranks
    rng = np.random.default_rng(1)
    for _ in range(50):
        B = int(rng.integers(1, 5))
        wins = [rng.integers(1, 65, int(rng.integers(1, 9))).tolist() for _ in range(B)]
        lengths = [sum(w) for w in wins]
        cu = np.concatenate([[0], np.cumsum([x for w in wins for x in w])]).tolist()
        for sp in (1, 2, 3, 4, 7):
            for r in range(sp):
                for cuw in (None, cu):
                    slices, wr, _ = sp_oracle.split_slices(lengths, r, sp, cuw)
                    meta = spu.plan_split(lengths, r, sp, cu_window_seqlens=None if cuw is None else torch.tensor(cuw))
                    assert meta.sample_global_slices == slices and meta.window_index_ranges == wr
            total = sum(spu.plan_split(lengths, r, sp, cu_window_seqlens=torch.tensor(cu)).total_local_len for r in range(sp))
            assert total == sum(lengths)


def test_oracle_split_pad_reinterleave_roundtrip():
    rng = np.random.default_rng(2)
    lengths = [10, 14, 3]
    x = rng.standard_normal((27, 5)).astype(np.float32)
    for sp in (1, 2, 3, 5):
        packs = [sp_oracle.split_rows(x, lengths, r, sp) for r in range(sp)]
        lm = np.array([[b - a for a, b in sp_oracle.split_slices(lengths, r, sp)[0]] for r in range(sp)])
        assert np.array_equal(sp_oracle.reinterleave(packs, lm), x)
    padded, mask = sp_oracle.pad_rows(x[:8], [3, 5], pad_value=-999.0)
    assert padded.shape == (2, 5, 5) and (padded[0, 3:] == -999.0).all() and mask[0].tolist() == [True] * 3 + [False] * 2
    back, lens = sp_oracle.unpad(padded, mask)
    assert np.array_equal(back, x[:8]) and lens == [3, 5]
    with pytest.raises(ValueError):
        sp_oracle.pad_rows(x[:8], [3, 5], pad_to=4)
    assert sp_oracle.unpad(padded, np.zeros_like(mask))[0].shape[0] == 0
