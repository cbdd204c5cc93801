"""Parity of every HIP kernel (called through the C ABI) against the CPU oracle.

Tolerances (max |a-b| / max |b|): 1e-4 in fp32, 2e-2 in bf16; index / copy kernels are bit-exact.
"""

import math

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle import sp_oracle, vit_oracle
from oracle.vit_oracle import max_rel_err

pytestmark = pytest.mark.gpu

TOL = {torch.float32: 1e-4, torch.bfloat16: 2e-2}
DEV = "cuda:0"


def _ops():
    from mi355_vit import ops

    return ops


def _rand(shape, dtype, seed, scale=1.0):
    g = torch.Generator(device="cpu").manual_seed(seed)
    return (torch.randn(*shape, generator=g) * scale).to(dtype)


def _announce(msg):
    print(f"[case] {msg}", flush=True)


# ------------------------------------------------------------------------------------------ RMSNorm
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("rows,cols", [(512, 1280), (37, 256), (5, 100), (4096, 1280)])
def test_rmsnorm_fwd_bwd(dtype, rows, cols):
    _announce(f"rmsnorm {dtype} {rows}x{cols}")
    ops = _ops()
    x = _rand((rows, cols), dtype, 0)
    w = (1.0 + 0.1 * _rand((cols,), torch.float32, 1)).to(dtype)
    dy = _rand((rows, cols), dtype, 2)
    add = _rand((rows, cols), dtype, 3)
    y, rstd = ops.rmsnorm_fwd(x.to(DEV), w.to(DEV), 1e-6)
    xr = x.float().requires_grad_(True)
    wr = w.float().requires_grad_(True)
    yr = vit_oracle.rms_norm(xr, wr, 1e-6)
    # the oracle formula itself is pinned against the library routine
    assert max_rel_err(yr, F.rms_norm(xr, (cols,), wr, 1e-6)) < 1e-6
    assert max_rel_err(y, yr) < TOL[dtype]
    yr.backward(dy.float())
    dx, dw = ops.rmsnorm_bwd(dy.to(DEV), x.to(DEV), w.to(DEV), rstd, dx_add=add.to(DEV))
    assert max_rel_err(dx, xr.grad + add.float()) < TOL[dtype]
    assert max_rel_err(dw, wr.grad) < TOL[dtype]
    dx2, _ = ops.rmsnorm_bwd(dy.to(DEV), x.to(DEV), w.to(DEV), rstd)
    assert max_rel_err(dx2, xr.grad) < TOL[dtype]


# ------------------------------------------------------------------------------------------ RoPE
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("S,H,d", [(300, 16, 80), (64, 8, 32), (17, 4, 6)])
def test_rope_fwd_bwd(dtype, S, H, d):
    _announce(f"rope {dtype} S={S} H={H} d={d}")
    ops = _ops()
    pad = 8 if d % 8 == 0 else 0
    x = _rand((S, H * d + pad * d), dtype, 0)  # extra columns must stay untouched
    ang = _rand((S, d), torch.float32, 1, 3.0)  # deliberately different halves: the general form
    cos, sin = ang.cos(), ang.sin()
    xg = x.to(DEV).clone()
    ops.rope_(xg, cos.to(DEV), sin.to(DEV), H, d)
    ref = vit_oracle.rope_apply(x[:, : H * d].reshape(S, H, d), cos, sin).reshape(S, H * d)
    assert max_rel_err(xg[:, : H * d], ref.float()) < TOL[dtype]
    assert torch.equal(xg[:, H * d :].cpu(), x[:, H * d :])
    # closed form: every (j, j+d/2) pair is rotated when both halves share the angle -> norms are preserved
    a2 = torch.cat([ang[:, : d // 2]] * 2, dim=-1)
    xf = _rand((S, H * d), torch.float32, 5)
    xr = xf.to(DEV).clone()
    ops.rope_(xr, a2.cos().to(DEV), a2.sin().to(DEV), H, d)
    n0 = xf.view(S, H, 2, d // 2).pow(2).sum(2)
    n1 = xr.cpu().view(S, H, 2, d // 2).pow(2).sum(2)
    assert torch.allclose(n0, n1, rtol=1e-4, atol=1e-5)
    # backward = transpose of the forward map
    xin = x[:, : H * d].float().reshape(S, H, d).requires_grad_(True)
    g = _rand((S, H * d), dtype, 7)
    vit_oracle.rope_apply(xin, cos, sin).backward(g.float().reshape(S, H, d))
    gg = g.to(DEV).clone()
    ops.rope_(gg, cos.to(DEV), sin.to(DEV), H, d, backward=True)
    assert max_rel_err(gg, xin.grad.reshape(S, H * d)) < TOL[dtype]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_rope_with_scaled_leading_heads(dtype):
    """The first `lead_heads` heads leave the rotary pass multiplied by `lead_scale`, in the same rounding: bit-equal to
    the oracle's rotation times the factor rounded once; the other heads and the columns behind them as without it."""
    _announce(f"rope with scaled leading heads {dtype}")
    ops = _ops()
    S, H, d, lead, gain = 300, 6, 80, 3, 0.1613
    x = _rand((S, H * d + 16), dtype, 0)
    ang = torch.cat([_rand((S, d // 2), torch.float32, 1, 3.0)] * 2, dim=-1)
    cos, sin = ang.cos(), ang.sin()
    for backward in (False, True):
        got = x.to(DEV).clone()
        ops.rope_(got, cos.to(DEV), sin.to(DEV), H, d, backward=backward, lead_heads=lead, lead_scale=gain)
        plain = x.to(DEV).clone()
        ops.rope_(plain, cos.to(DEV), sin.to(DEV), H, d, backward=backward)
        assert torch.equal(got[:, lead * d :], plain[:, lead * d :])
        xin = x[:, : H * d].float().reshape(S, H, d).requires_grad_(backward)
        if backward:
            vit_oracle.rope_apply(xin, cos, sin).backward(x[:, : H * d].float().reshape(S, H, d))
            rot = xin.grad
        else:
            rot = vit_oracle.rope_apply(xin, cos, sin)
        want = (rot[:, :lead] * torch.tensor(gain, dtype=torch.float32)).reshape(S, lead * d)
        assert max_rel_err(got[:, : lead * d], want) < (1e-6 if dtype == torch.float32 else 2.0**-8)


def test_queries_scaled_in_the_rotary_pass_are_rounded_once():
    """What the block does (queries take head_dim^-1/2 * log2 e in the rotary pass, attention called with scale
    1 / log2 e) against handing bf16 queries to the attention entry point with the plain scale (which rounds q * scale
    to bf16 a second time): with scores of standard deviation 9 the output error against float64 attention on the
    unrounded queries falls from 2.5e-2 to 1.5e-2, the level of exact attention on queries rounded once."""
    _announce("attention: queries scaled in the rotary pass")
    ops = _ops()
    S, H, d, LOG2E = 2048, 4, 80, 1.4426950408889634
    g = torch.Generator().manual_seed(0)
    q32 = torch.randn(S, H * d, generator=g) * 3.0  # fp32 queries as they leave the rotation, before any rounding
    k = (torch.randn(S, H * d, generator=g) * 3.0).to(torch.bfloat16)
    v = torch.randn(S, H * d, generator=g).to(torch.bfloat16)
    cu = torch.tensor([0, S], dtype=torch.int32, device=DEV)
    heads = lambda t: t.double().to(DEV).reshape(S, H, d).transpose(0, 1)  # noqa: E731
    ref = (torch.softmax(heads(q32) @ heads(k).transpose(1, 2) * d**-0.5, -1) @ heads(v)).transpose(0, 1).reshape(S, H * d)
    err = lambda o: float((o.double() - ref).abs().max() / ref.abs().max())  # noqa: E731
    twice, _ = ops.attn_fwd(q32.to(torch.bfloat16).to(DEV), k.to(DEV), v.to(DEV), cu, S, H, d, d**-0.5)
    once, _ = ops.attn_fwd((q32 * (d**-0.5 * LOG2E)).to(torch.bfloat16).to(DEV), k.to(DEV), v.to(DEV), cu, S, H, d, 1.0 / LOG2E)
    # float64 attention on queries rounded to bf16 once, everything else exact: what no bf16 pipeline can beat by much
    floor = err((torch.softmax(heads(q32.to(torch.bfloat16)) @ heads(k).transpose(1, 2) * d**-0.5, -1) @ heads(v)).transpose(0, 1).reshape(S, H * d))
    e_twice, e_once = err(twice), err(once)
    print(f"    output error: q rounded, then q * scale rounded {e_twice:.2e}; q * scale rounded once {e_once:.2e}; "
          f"exact attention on once-rounded q {floor:.2e}", flush=True)
    assert e_once < 2e-2 and e_once < 0.75 * e_twice and e_once < 1.5 * floor


@pytest.mark.parametrize("late_key", [40, 1500, 2047])
def test_attention_forward_scores_far_above_the_first_tiles(late_key):
    """The long-segment forward sets its stabiliser from the first tile of keys and leaves it there; a later score that
    exceeds it by more than the exponent range of exp2 overflows the row's sums, which the kernel sees at the end and
    answers with a second sweep that follows the maxima tile by tile.  Here one late key scores about 190 base-2 units
    above everything before it for every query: the result must still be the exact softmax (all weight on that key)."""
    _announce(f"attention fwd: a score 190 binary orders above the first tile's maximum at key {late_key}")
    ops = _ops()
    S, H, d = 2048, 2, 80
    g = torch.Generator().manual_seed(5)
    u = torch.randn(H, d, generator=g)
    u = u / u.norm(dim=1, keepdim=True)
    q = (34.0 * u[None] + 0.1 * torch.randn(S, H, d, generator=g)).reshape(S, H * d).to(torch.bfloat16)
    k = 0.1 * torch.randn(S, H, d, generator=g)
    k[late_key] = 34.0 * u
    k = k.reshape(S, H * d).to(torch.bfloat16)
    v = torch.randn(S, H * d, generator=g).to(torch.bfloat16)
    cu = torch.tensor([0, S], dtype=torch.int32, device=DEV)
    o, lse = ops.attn_fwd(q.to(DEV), k.to(DEV), v.to(DEV), cu, S, H, d, d**-0.5)
    heads = lambda t: t.double().reshape(S, H, d).transpose(0, 1)  # noqa: E731
    scores = heads(q) @ heads(k).transpose(1, 2) * d**-0.5
    assert float((scores[:, :, late_key] - scores[:, :, :32].amax(-1)).min()) * 1.4427 > 150.0  # the case is what it says
    ref = (torch.softmax(scores, -1) @ heads(v)).transpose(0, 1).reshape(S, H * d)
    assert torch.isfinite(o).all() and torch.isfinite(lse).all()
    assert max_rel_err(o, ref) < TOL[torch.bfloat16]
    assert max_rel_err(lse, torch.logsumexp(scores, -1)) < 5e-3  # the kernel rounds q * scale to bf16: 2^-9 of a score of 129
    # the ordinary case next to it on the same launch shape: nothing overflows, one sweep
    k2 = (0.1 * torch.randn(S, H * d, generator=g)).to(torch.bfloat16)
    o2, _ = ops.attn_fwd(q.to(DEV), k2.to(DEV), v.to(DEV), cu, S, H, d, d**-0.5)
    ref2 = (torch.softmax(heads(q) @ heads(k2).transpose(1, 2) * d**-0.5, -1) @ heads(v)).transpose(0, 1).reshape(S, H * d)
    assert max_rel_err(o2, ref2) < TOL[torch.bfloat16]


# ------------------------------------------------------------------------------------------ copies
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_gather_rows_window_permutation_bit_exact(dtype):
    ops = _ops()
    grid = torch.tensor([[1, 18, 22], [2, 8, 12], [1, 16, 16]])
    widx, cu = ops.window_index(grid, 2, 112, 14)
    S = int((grid[:, 0] * grid[:, 1] * grid[:, 2]).sum())
    x = _rand((S, 1280), dtype, 0)
    out = ops.gather_rows(x.to(DEV), widx.to(DEV), 4).cpu()
    ref = x.view(S // 4, 4, -1)[widx].reshape(S, -1)
    assert torch.equal(out.view(torch.int16 if dtype == torch.bfloat16 else torch.int32), ref.view(torch.int16 if dtype == torch.bfloat16 else torch.int32))
    rev = torch.argsort(widx)
    back = ops.gather_rows(out.to(DEV), rev.to(DEV), 4).cpu()
    assert torch.equal(back.view(torch.int32 if dtype == torch.float32 else torch.int16), x.view(torch.int32 if dtype == torch.float32 else torch.int16))
    # odd row width (falls back to 4-byte words)
    y = _rand((12, 6), dtype, 1)
    perm = torch.randperm(12, generator=torch.Generator().manual_seed(0))
    assert torch.equal(ops.gather_rows(y.to(DEV), perm.to(DEV)).cpu(), y[perm])


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("sp", [1, 2, 3, 4, 8])
def test_split_gather_bit_exact(dtype, sp):
    """split_pack_by_sp for every rank, then the re-interleave: must reproduce the input bit for bit."""
    from mi355_vit import sequence_parallel_utils as spu

    ops = _ops()
    g = torch.Generator().manual_seed(2)
    hw = 2 * torch.randint(4, 20, (5, 2), generator=g)
    grid = torch.cat([torch.ones(5, 1, dtype=torch.long), hw], dim=1)
    grid[1, 0] = 2
    _, cu_w = ops.window_index(grid, 2, 112, 14)
    lengths = (ops.cu_seqlens(grid)[1:] - ops.cu_seqlens(grid)[:-1]).tolist()
    S = sum(lengths)
    x = _rand((S, 320), dtype, 3)
    xg = x.to(DEV)
    for windows in (None, cu_w):
        packs, metas = [], []
        for r in range(sp):
            pk, meta = spu.split_pack_by_sp(xg, lengths, r, sp, cu_window_seqlens=windows)
            ref = sp_oracle.split_rows(x.view(torch.int16 if dtype == torch.bfloat16 else torch.int32).numpy(), lengths, r, sp,
                                       None if windows is None else windows.tolist())
            assert np.array_equal(pk.cpu().view(torch.int16 if dtype == torch.bfloat16 else torch.int32).numpy(), ref)
            packs.append(pk)
            metas.append(meta)
        lm = [m.local_lengths for m in metas]
        rebuilt = spu.gather_rank_packs(packs, lm)
        assert torch.equal(rebuilt.cpu().view(torch.uint8), x.view(torch.uint8))
        assert sum(m.total_local_len for m in metas) == S


def test_split_gather_with_empty_rank_shares():
    """Samples shorter than the sequence-parallel degree (4-patch images, sp = 8): some ranks receive nothing from a sample,
    some nothing at all; packs of zero rows travel through split, pad / unpad and the re-interleave like any other."""
    from mi355_vit import sequence_parallel_utils as spu

    for lengths, sp, some_rank_empty in (([4, 4, 16, 4], 8, False), ([4, 4, 16, 4], 5, False), ([4, 2, 4], 8, True)):
        S = sum(lengths)
        x = _rand((S, 64), torch.bfloat16, 7)
        xg = x.to(DEV)
        _announce(f"split/gather with empty shares lengths={lengths} sp={sp}")
        packs, metas = [], []
        for r in range(sp):
            pk, meta = spu.split_pack_by_sp(xg, lengths, r, sp)
            ref = sp_oracle.split_rows(x.view(torch.int16).numpy(), lengths, r, sp, None)
            assert pk.shape[0] == ref.shape[0] and np.array_equal(pk.cpu().view(torch.int16).numpy().reshape(ref.shape), ref)
            padded, mask = spu.pad_pack_to_batch(pk, meta, pad_value=-999.0, enforce_min_pad=1)
            assert padded.shape[:2] == (len(lengths), max(1, meta.max_local_len)) and mask.sum(dim=1).tolist() == list(meta.local_lengths)
            back, _ = spu.unpad_batch_to_pack(padded, mask)
            assert torch.equal(back.view(torch.int16), pk.view(torch.int16))
            packs.append(pk)
            metas.append(meta)
        assert any(0 in m.local_lengths for m in metas)
        assert any(m.total_local_len == 0 for m in metas) == some_rank_empty
        rebuilt = spu.gather_rank_packs(packs, [m.local_lengths for m in metas])
        assert torch.equal(rebuilt.cpu().view(torch.uint8), x.view(torch.uint8))


def test_split_gather_sp4_real_shape():
    """Five square images with sides drawn from the multiples of 28 in [448, 3584] (seed 2), hidden 1280, bf16,
    split into 4 sequence-parallel shards (token cuts and window-aligned cuts) and gathered back: bit-exact."""
    from mi355_vit import sequence_parallel_utils as spu

    ops = _ops()
    g = torch.Generator().manual_seed(2)
    side = 2 * torch.randint(16, 129, (5,), generator=g)  # patches per side (even: 28 px = 2 patches)
    grid = torch.stack([torch.ones(5, dtype=torch.long), side, side], dim=1)
    _, cu_w = ops.window_index(grid, 2, 112, 14)
    lengths = (side * side).tolist()
    S = sum(lengths)
    _announce(f"split/gather real shape: {S} patches")
    xg = torch.randint(-32768, 32767, (S, 1280), dtype=torch.int16, generator=g).view(torch.bfloat16).to(DEV)
    x_np = xg.cpu().view(torch.int16).numpy()
    for windows in (None, cu_w):
        packs, metas = [], []
        for r in range(4):
            pk, meta = spu.split_pack_by_sp(xg, lengths, r, 4, cu_window_seqlens=windows)
            ref = sp_oracle.split_rows(x_np, lengths, r, 4, None if windows is None else windows.tolist())
            assert np.array_equal(pk.cpu().view(torch.int16).numpy(), ref)
            packs.append(pk)
            metas.append(meta)
        rebuilt = spu.gather_rank_packs(packs, [m.local_lengths for m in metas])
        assert torch.equal(rebuilt.view(torch.int16), xg.view(torch.int16))
        if windows is None:
            assert max(m.total_local_len for m in metas) - min(m.total_local_len for m in metas) <= len(lengths)


def test_split_gather_reference_sizes():
    """tests/test_split_gather.py of the reference: arange tensors of 1024 and 1020 rows x 1280, two ranks."""
    from mi355_vit import sequence_parallel_utils as spu

    for rows in (1024, 1020):
        x = torch.arange(rows * 1280, dtype=torch.float32).reshape(rows, 1280).to(DEV)
        packs, lm = [], []
        for r in range(2):
            pk, meta = spu.split_pack_by_sp(x, [rows], r, 2)
            packs.append(pk)
            lm.append(meta.local_lengths)
        assert packs[0].shape[0] == rows // 2
        assert torch.equal(packs[0], x[: rows // 2])
        assert torch.equal(spu.gather_rank_packs(packs, lm), x)


def test_pad_unpad_and_local_rope():
    from mi355_vit import sequence_parallel_utils as spu

    x = _rand((20, 64), torch.bfloat16, 0).to(DEV)
    pk, meta = spu.split_pack_by_sp(x, [12, 8], 0, 2)
    assert meta.local_lengths == [6, 4]
    padded, mask = spu.pad_pack_to_batch(pk, meta, pad_value=-999.0)
    assert padded.shape == (2, 6, 64) and mask.dtype == torch.bool
    assert mask[0].all() and mask[1, :4].all() and not mask[1, 4:].any()
    assert (padded[1, 4:] == -999.0).all()
    pad_bf16 = torch.tensor(-999.0, dtype=torch.bfloat16).float().item()  # the pad value as bf16 stores it
    ref, rmask = sp_oracle.pad_rows(pk.cpu().float().numpy(), [6, 4], pad_value=pad_bf16)
    assert np.array_equal(padded.cpu().float().numpy(), ref) and np.array_equal(mask.cpu().numpy(), rmask)
    back, lens = spu.unpad_batch_to_pack(padded, mask, return_lengths=True)
    assert lens == [6, 4] and torch.equal(back, pk)
    p2, m2 = spu.pad_pack_to_batch(pk, meta, pad_to=9, enforce_min_pad=1)
    assert p2.shape == (2, 9, 64)
    with pytest.raises(ValueError):
        spu.pad_pack_to_batch(pk, meta, pad_to=3)
    empty, _ = spu.unpad_batch_to_pack(torch.randn(2, 5, 32, device=DEV), torch.zeros(2, 5, dtype=torch.bool, device=DEV))
    assert empty.shape == (0, 32)
    cos, sin = torch.randn(20, 32, device=DEV), torch.randn(20, 32, device=DEV)
    c0, s0, m0 = spu.build_local_rope(meta, cos, sin)
    assert m0 is None and torch.equal(c0[:6], cos[0:6]) and torch.equal(c0[6:10], cos[12:16]) and torch.equal(s0[6:], sin[12:16])
    cp, sp_, mk = spu.build_local_rope(meta, cos, sin, pad_to=7)
    assert cp.shape == (2, 7, 32) and mk.shape == (2, 7) and (cp[1, 4:] == 0).all() and torch.equal(cp[0, :6], cos[:6])


def test_cast2d_and_colsum():
    ops = _ops()
    x = _rand((300, 70), torch.float32, 0)
    dst = torch.zeros(300, 96, dtype=torch.bfloat16, device=DEV)
    ops.cast2d(x.to(DEV), dst[:, 8:78])
    assert torch.equal(dst[:, 8:78].cpu(), x.to(torch.bfloat16)) and (dst[:, :8] == 0).all() and (dst[:, 78:] == 0).all()
    for dtype in (torch.float32, torch.bfloat16):
        y = _rand((1000, 130), dtype, 1)
        s = ops.colsum(y.to(DEV)[:, 1:129], torch.float32)
        assert max_rel_err(s, y[:, 1:129].float().sum(0)) < 1e-5


# ------------------------------------------------------------------------------------------ GEMM
def _gemm_ref(a, b):
    return a.double() @ b.double().t()


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("M,N,K", [(512, 1280, 1280), (300, 200, 72), (1000, 3424, 1280), (260, 1280, 1176), (8, 8, 8)])
def test_gemm_plain_bias_residual(dtype, M, N, K):
    _announce(f"gemm NT {dtype} {M}x{N}x{K}")
    ops = _ops()
    from mi355_vit import _lib as E

    a, b = _rand((M, K), dtype, 0), _rand((N, K), dtype, 1, K**-0.5)
    bias, res = _rand((N,), dtype, 2), _rand((M, N), dtype, 3)
    ref = _gemm_ref(a, b)
    out = torch.empty(M, N, dtype=dtype, device=DEV)
    ops.gemm(a.to(DEV), b.to(DEV), out)
    assert max_rel_err(out, ref) < TOL[dtype]
    ops.gemm(a.to(DEV), b.to(DEV), out, epilogue=E.EPI_BIAS, bias=bias.to(DEV))
    assert max_rel_err(out, ref + bias.double()) < TOL[dtype]
    ops.gemm(a.to(DEV), b.to(DEV), out, epilogue=E.EPI_BIAS_RES, bias=bias.to(DEV), residual=res.to(DEV))
    assert max_rel_err(out, ref + bias.double() + res.double()) < TOL[dtype]
    ops.gemm(a.to(DEV), b.to(DEV), out, epilogue=E.EPI_ACCUM)
    assert max_rel_err(out, 2 * ref + bias.double() + res.double()) < TOL[dtype]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("M,N,K", [(512, 1280, 3840), (300, 200, 72), (130, 1280, 6848), (257, 3420, 1280)])
def test_gemm_dgrad_layout(dtype, M, N, K):
    """C = A . W with W stored [K, N] (the weight as it lies in memory): trans_b."""
    _announce(f"gemm NN {dtype} {M}x{N}x{K}")
    ops = _ops()
    a, w = _rand((M, K), dtype, 0), _rand((K, (N + 7) // 8 * 8), dtype, 1, K**-0.5)
    out = torch.empty(M, N, dtype=dtype, device=DEV)
    ops.gemm(a.to(DEV), w.to(DEV), out, trans_b=True, n=N)
    assert max_rel_err(out, a.double() @ w.double()[:, :N]) < TOL[dtype]


@pytest.mark.parametrize("M", [4096, 16384, 1000, 130, 3408])
@pytest.mark.parametrize("K", [1280, 3424])
def test_gemm_half_height_tiles_give_the_same_bits_as_full_tiles(M, K, monkeypatch):
    """Products with few tile columns (N = 1280) take 128-row tiles when 256-row tiles would leave most compute units
    idle.  The choice follows M, so it must not change a single bit: same K order, same MFMA form, same epilogue."""
    _announce(f"gemm half tiles M={M} K={K}")
    ops = _ops()
    from mi355_vit import _lib as E

    N, dtype = 1280, torch.bfloat16
    a, b = _rand((M, K), dtype, 0).to(DEV), _rand((N, K), dtype, 1, K**-0.5).to(DEV)
    w = _rand((K, N), dtype, 4, K**-0.5).to(DEV)
    bias, res = _rand((N,), dtype, 2).to(DEV), _rand((M, N), dtype, 3).to(DEV)

    def run():
        fwd = torch.full((M, N), 7.0, dtype=dtype, device=DEV)
        dgrad = torch.full((M, N), 7.0, dtype=dtype, device=DEV)
        ops.gemm(a, b, fwd, epilogue=E.EPI_BIAS_RES, bias=bias, residual=res)
        ops.gemm(a, w, dgrad, trans_b=True)
        torch.cuda.synchronize()
        return fwd, dgrad

    monkeypatch.setenv("MVIT_GEMM_NO_HALF_TILES", "1")
    fwd_full, dgrad_full = run()
    monkeypatch.delenv("MVIT_GEMM_NO_HALF_TILES")
    fwd_half, dgrad_half = run()
    assert torch.equal(fwd_half, fwd_full) and torch.equal(dgrad_half, dgrad_full)
    assert max_rel_err(fwd_half, _gemm_ref(a.cpu(), b.cpu()) + bias.cpu().double() + res.cpu().double()) < TOL[dtype]
    assert max_rel_err(dgrad_half, a.cpu().double() @ w.cpu().double()) < TOL[dtype]


@pytest.mark.parametrize("dtype,odt", [(torch.float32, torch.float32), (torch.bfloat16, torch.bfloat16), (torch.bfloat16, torch.float32)])
@pytest.mark.parametrize("S,No,Ni", [(1000, 1280, 1280), (515, 3840, 256), (70, 6848, 1280), (2052, 1280, 3420)])
def test_gemm_wgrad_layout(dtype, odt, S, No, Ni):
    """dW[No, Ni] = dY^T . X with dY [S, No] and X [S, Ni] as they lie in memory: trans_a and trans_b."""
    _announce(f"gemm TT {dtype}->{odt} S={S} {No}x{Ni}")
    ops = _ops()
    ldx = (Ni + 7) // 8 * 8
    dy, x = _rand((S, No), dtype, 0), _rand((S, ldx), dtype, 1)
    out = torch.empty(No, Ni, dtype=odt, device=DEV)
    ops.gemm(dy.to(DEV), x.to(DEV), out, trans_a=True, trans_b=True, n=Ni)
    assert max_rel_err(out, dy.double().t() @ x.double()[:, :Ni]) < TOL[dtype]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_gemm_gelu_and_swiglu_epilogues(dtype):
    ops = _ops()
    from mi355_vit import _lib as E

    M, K, N = 384, 640, 520
    a = _rand((M, K), dtype, 0)
    w, b = _rand((N, K), dtype, 1, K**-0.5), _rand((N,), dtype, 2)
    z = torch.empty(M, N, dtype=dtype, device=DEV)
    y = torch.empty_like(z)
    ops.gemm(a.to(DEV), w.to(DEV), y, epilogue=E.EPI_BIAS_GELU, bias=b.to(DEV), aux=z)
    zr = F.linear(a.float(), w.float(), b.float())
    assert max_rel_err(z, zr) < TOL[dtype]
    assert max_rel_err(y, F.gelu(z.float().cpu())) < TOL[dtype]  # gelu of the stored pre-activation
    # gelu backward epilogue: dz = (dy . W2) * gelu'(z)
    O = 264
    dy, w2 = _rand((M, O), dtype, 3), _rand((O, N), dtype, 4, N**-0.5)
    dz = torch.empty(M, N, dtype=dtype, device=DEV)
    ops.gemm(dy.to(DEV), w2.to(DEV), dz, trans_b=True, epilogue=E.EPI_GELU_BWD, residual=z)
    zc = z.float().cpu().requires_grad_(True)
    F.gelu(zc).backward(dy.float() @ w2.float())
    assert max_rel_err(dz, zc.grad) < TOL[dtype]

    # SwiGLU: packed [2*Ipad, K] weight with zero padding rows, as the block uses it
    I, Ipad = 516, 520
    wg, wu = _rand((I, K), dtype, 5, K**-0.5), _rand((I, K), dtype, 6, K**-0.5)
    bg, bu = _rand((I,), dtype, 7), _rand((I,), dtype, 8)
    wgu = torch.zeros(2 * Ipad, K, dtype=dtype)
    wgu[:I], wgu[Ipad : Ipad + I] = wg, wu
    bgu = torch.zeros(2 * Ipad, dtype=dtype)
    bgu[:I], bgu[Ipad : Ipad + I] = bg, bu
    wgu, bgu = wgu.to(DEV), bgu.to(DEV)
    gu = torch.full((M, 2 * Ipad), float("nan"), dtype=dtype, device=DEV)
    h = torch.full((M, Ipad), float("nan"), dtype=dtype, device=DEV)
    ops.gemm(a.to(DEV), wgu[:Ipad], h, epilogue=E.EPI_SWIGLU, b2=wgu[Ipad:], bias=bgu[:Ipad], bias2=bgu[Ipad:], aux=gu, aux_off=Ipad)
    gr, ur = F.linear(a.float(), wg.float(), bg.float()), F.linear(a.float(), wu.float(), bu.float())
    assert max_rel_err(gu[:, :I], gr) < TOL[dtype] and max_rel_err(gu[:, Ipad : Ipad + I], ur) < TOL[dtype]
    assert max_rel_err(h[:, :I], F.silu(gr) * ur) < TOL[dtype]
    assert (h[:, I:] == 0).all() and (gu[:, I:Ipad] == 0).all() and (gu[:, Ipad + I :] == 0).all()
    # without aux (a forward that will not be differentiated): the same product, bit for bit, and nothing else written
    h_only = torch.full((M, Ipad), float("nan"), dtype=dtype, device=DEV)
    ops.gemm(a.to(DEV), wgu[:Ipad], h_only, epilogue=E.EPI_SWIGLU, b2=wgu[Ipad:], bias=bgu[:Ipad], bias2=bgu[Ipad:], aux_off=Ipad)
    assert torch.equal(h_only.view(torch.uint8), h.view(torch.uint8))
    # backward epilogue: (dg, du) from dh = dx . Wdown, Wdown stored [C, Ipad] with zero padding columns
    Cc = 256
    dx, wd = _rand((M, Cc), dtype, 9), torch.zeros(Cc, Ipad, dtype=dtype)
    wd[:, :I] = _rand((Cc, I), dtype, 10, I**-0.5)
    dgu = torch.full((M, 2 * Ipad), float("nan"), dtype=dtype, device=DEV)
    part = torch.full((-(-M // 256), 2 * Ipad), float("nan"), dtype=torch.float32, device=DEV)
    ops.gemm(dx.to(DEV), wd.to(DEV), dgu, trans_b=True, epilogue=E.EPI_SWIGLU_BWD, residual=gu, aux_off=Ipad, colsum_partial=part)
    # fused bias gradient: column sums of dgu, accumulated in fp32 before the rounding to the storage type
    bsum = ops.reduce_partials(part, torch.float32)
    assert max_rel_err(bsum, dgu.float().sum(0)) < TOL[dtype]
    g0 = gu[:, :I].float().cpu().requires_grad_(True)
    u0 = gu[:, Ipad : Ipad + I].float().cpu().requires_grad_(True)
    (F.silu(g0) * u0).backward(dx.float() @ wd.float()[:, :I])
    assert max_rel_err(dgu[:, :I], g0.grad) < TOL[dtype] and max_rel_err(dgu[:, Ipad : Ipad + I], u0.grad) < TOL[dtype]
    assert (dgu[:, I:Ipad] == 0).all() and (dgu[:, Ipad + I :] == 0).all()


# ------------------------------------------------------------------------------------------ attention
def _attn_case(dtype, seglens, H, d, seed=0, qkv_packed=True):
    ops = _ops()
    S = sum(seglens)
    cu = torch.tensor([0] + list(np.cumsum(seglens)), dtype=torch.int32)
    if qkv_packed:  # q, k, v are column blocks of one [S, 3*H*d] buffer, as in the block
        qkv = _rand((S, 3 * H * d), dtype, seed)
        q, k, v = qkv[:, : H * d], qkv[:, H * d : 2 * H * d], qkv[:, 2 * H * d :]
        qkvg = qkv.to(DEV)
        qg, kg, vg = qkvg[:, : H * d], qkvg[:, H * d : 2 * H * d], qkvg[:, 2 * H * d :]
    else:
        q, k, v = (_rand((S, H * d), dtype, seed + i) for i in range(3))
        qg, kg, vg = q.to(DEV), k.to(DEV), v.to(DEV)
    do = _rand((S, H * d), dtype, seed + 7)
    scale = d**-0.5
    og, lse = ops.attn_fwd(qg, kg, vg, cu.to(DEV), max(seglens), H, d, scale)
    qr, kr, vr = (t.float().reshape(S, H, d).clone().requires_grad_(True) for t in (q, k, v))
    oref = vit_oracle.attention(qr, kr, vr, cu)
    # pin the oracle's attention against the library routine on the first segment
    L0 = seglens[0]
    if L0:
        sd = F.scaled_dot_product_attention(qr[:L0].transpose(0, 1)[None], kr[:L0].transpose(0, 1)[None], vr[:L0].transpose(0, 1)[None])
        assert max_rel_err(oref[:L0], sd[0].transpose(0, 1)) < 1e-5
    assert max_rel_err(og, oref.reshape(S, H * d)) < TOL[dtype], "forward"
    lse_ref = []
    for a, b in zip(cu[:-1].tolist(), cu[1:].tolist()):
        s = torch.einsum("qhd,khd->hqk", qr[a:b], kr[a:b]) * scale
        lse_ref.append(torch.logsumexp(s, dim=-1))
    assert torch.allclose(lse.cpu(), torch.cat(lse_ref, dim=1).detach(), rtol=2e-3 if dtype == torch.bfloat16 else 1e-5, atol=2e-3 if dtype == torch.bfloat16 else 1e-5)
    oref.backward(do.float().reshape(S, H, d))
    dq, dk, dv = (torch.empty(S, H * d, dtype=dtype, device=DEV) for _ in range(3))
    ops.attn_bwd(qg, kg, vg, og, do.to(DEV), lse, cu.to(DEV), max(seglens), H, d, scale, dq, dk, dv)
    for name, got, ref in (("dq", dq, qr.grad), ("dk", dk, kr.grad), ("dv", dv, vr.grad)):
        assert max_rel_err(got, ref.reshape(S, H * d)) < TOL[dtype], name


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize(
    "seglens,H,d",
    [
        ([64] * 6, 16, 80),  # windows
        ([64, 16, 48, 64, 32, 4], 4, 80),  # ragged edge windows
        ([1, 17, 63, 33, 5], 2, 80),  # short windows of odd lengths (fused window backward)
        ([64, 20, 40], 2, 64),
        ([40, 64, 7], 2, 32),
        ([256, 256], 16, 80),  # cfg-1 full layer
        ([300, 77, 1, 130], 2, 80),  # ragged, single-token segment
        ([100, 60], 8, 32),
        ([129], 2, 64),
        ([96, 200], 2, 128),
        ([65, 128, 127], 2, 80),  # either side of the 64- and 128-token kernel choices
        ([511, 2], 2, 80),  # one token below the long-segment kernels
        # long segments (the 64-rows-per-wave backward kernels): tile multiples, tails of 1 / 31 / 33 rows, short
        # segments riding in the same launch
        ([512], 2, 80),
        ([513, 543], 2, 80),
        ([576, 1000, 33, 1], 4, 80),
        ([1200, 77, 640, 607], 3, 80),
    ],
)
def test_attention_fwd_bwd(dtype, seglens, H, d):
    _announce(f"attention {dtype} seglens={seglens} H={H} d={d}")
    _attn_case(dtype, seglens, H, d)


def test_attention_long_segment_bf16():
    """One 2,048-token segment with 4 heads (the sequence-parallel share shape, scaled down)."""
    _announce("attention bf16 long")
    _attn_case(torch.bfloat16, [2048, 1000], 4, 80, qkv_packed=False)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_attention_segment_order_changes_nothing(dtype):
    """seg_order only changes which work-group serves which segment: outputs and gradients are bit-identical with
    the natural order, the longest-first order of ops.segment_order and an arbitrary permutation; long (multi-block)
    and window-sized layouts."""
    ops = _ops()
    H, d = 4, 80
    for seglens in ([300, 1200, 77, 640, 1, 513], [64, 16, 48, 64]):
        _announce(f"attention seg_order {dtype} {seglens}")
        S = sum(seglens)
        cu = torch.tensor([0] + list(np.cumsum(seglens)), dtype=torch.int32).to(DEV)
        qkv = _rand((S, 3 * H * d), dtype, 5).to(DEV)
        q, k, v = qkv[:, : H * d], qkv[:, H * d : 2 * H * d], qkv[:, 2 * H * d :]
        do = _rand((S, H * d), dtype, 6).to(DEV)
        lf = ops.segment_order(torch.tensor(seglens))
        if max(seglens) > 64:
            assert lf.tolist() == sorted(range(len(seglens)), key=lambda i: -seglens[i])
        else:
            assert lf is None
        orders = [None, lf, torch.tensor(list(range(len(seglens)))[::-1], dtype=torch.int32)]
        res = []
        for order in orders:
            od = None if order is None else order.to(DEV)
            o, lse = ops.attn_fwd(q, k, v, cu, max(seglens), H, d, d**-0.5, seg_order=od)
            dq, dk, dv = (torch.full((S, H * d), float("nan"), dtype=dtype, device=DEV) for _ in range(3))
            ops.attn_bwd(q, k, v, o, do, lse, cu, max(seglens), H, d, d**-0.5, dq, dk, dv, seg_order=od)
            res.append((o, lse, dq, dk, dv))
        for other in res[1:]:
            for a, b in zip(res[0], other):
                assert torch.equal(a, b)
    with pytest.raises(ValueError):
        ops.attn_fwd(q, k, v, cu, 64, H, d, d**-0.5, seg_order=torch.zeros(2, dtype=torch.int32, device=DEV))


@pytest.mark.parametrize("H", [4, 16])
def test_attention_sp_share_real_shape(H):
    """One rank's share of Ulysses SP=4 attention at its real shape: 65,536 tokens, 4 of the 16 heads, head_dim 80
    (and, with 16 heads, the full-attention layer of the 65,536-patch image as the unsharded tower runs it).
    Windowed layout (64-token windows): everything against the oracle.  Full layer: the oracle's O(L^2) pass is
    out of reach on the host, so sampled query rows (O, lse, dQ) and sampled key rows (dK, dV) are recomputed in
    fp32 from their definitions; the key-row check takes lse and O for the non-sampled rows from the kernel."""
    ops = _ops()
    L, d = 65536, 80
    scale = d**-0.5
    if H == 4:
        _announce("attention bf16 SP share, windows")
        _attn_case(torch.bfloat16, [64] * 1024, H, d, seed=11)
    _announce(f"attention bf16 65,536 tokens x {H} heads, full layer")
    g = torch.Generator().manual_seed(12)
    q, k, v, do = (torch.randn(L, H * d, generator=g).to(torch.bfloat16).to(DEV) for _ in range(4))
    cu = torch.tensor([0, L], dtype=torch.int32, device=DEV)
    o, lse = ops.attn_fwd(q, k, v, cu, L, H, d, scale)
    dq, dk, dv = (torch.empty_like(q) for _ in range(3))
    ops.attn_bwd(q, k, v, o, do, lse, cu, L, H, d, scale, dq, dk, dv)
    idx = torch.randint(0, L, (48,), generator=g).to(DEV)
    qf, kf, vf, dof, of = (t.float().reshape(L, H, d) for t in (q, k, v, do, o))
    # sampled queries
    s = torch.einsum("qhd,khd->hqk", qf[idx], kf) * scale
    lse_ref = torch.logsumexp(s, dim=-1)  # [H, 48]
    p = torch.exp(s - lse_ref[..., None])
    o_ref = torch.einsum("hqk,khd->qhd", p, vf)
    assert max_rel_err(o[idx].float().reshape(-1, H, d), o_ref) < TOL[torch.bfloat16], "forward rows"
    assert torch.allclose(lse[:, idx], lse_ref, rtol=2e-3, atol=2e-3), "lse rows"
    dp = torch.einsum("qhd,khd->hqk", dof[idx], vf)
    delta = (dof[idx] * o_ref).sum(-1).transpose(0, 1)  # [H, 48]
    ds = p * (dp - delta[..., None])
    dq_ref = torch.einsum("hqk,khd->qhd", ds, kf) * scale
    assert max_rel_err(dq[idx].float().reshape(-1, H, d), dq_ref) < TOL[torch.bfloat16], "dq rows"
    # sampled keys
    st = torch.einsum("qhd,khd->hqk", qf, kf[idx]) * scale  # [H, L, 48]
    pt = torch.exp(st - lse[..., None])
    dv_ref = torch.einsum("hqk,qhd->khd", pt, dof)
    dpt = torch.einsum("qhd,khd->hqk", dof, vf[idx])
    delta_all = (dof * of).sum(-1).transpose(0, 1)  # [H, L]
    dk_ref = torch.einsum("hqk,qhd->khd", pt * (dpt - delta_all[..., None]), qf) * scale
    assert max_rel_err(dv[idx].float().reshape(-1, H, d), dv_ref) < TOL[torch.bfloat16], "dv rows"
    assert max_rel_err(dk[idx].float().reshape(-1, H, d), dk_ref) < TOL[torch.bfloat16], "dk rows"


def test_attention_softmax_invariants():
    """Properties that hold at any size: V constant -> O constant; outputs independent across segments."""
    ops = _ops()
    S, H, d = 700, 4, 80
    cu = torch.tensor([0, 300, 700], dtype=torch.int32, device=DEV)
    q, k = (_rand((S, H * d), torch.bfloat16, i).to(DEV) for i in range(2))
    v = torch.ones(S, H * d, dtype=torch.bfloat16, device=DEV) * 0.5
    o, _ = ops.attn_fwd(q, k, v, cu, 400, H, d, d**-0.5)
    assert torch.allclose(o.float(), torch.full_like(o.float(), 0.5), atol=4e-3)
    v2 = _rand((S, H * d), torch.bfloat16, 5).to(DEV)
    o1, _ = ops.attn_fwd(q, k, v2, cu, 400, H, d, d**-0.5)
    k2, v3 = k.clone(), v2.clone()
    k2[300:] = 0
    v3[300:] = 1
    o2, _ = ops.attn_fwd(q, k2, v3, cu, 400, H, d, d**-0.5)
    assert torch.equal(o1[:300], o2[:300])


def test_gemm_bf16_with_a_row_pitch_beyond_32_bit_lane_offsets():
    """Operands whose rows lie more than 2^22 elements apart take the register-staged bf16 main loop (the direct
    global -> LDS loads address a tile with 32-bit lane offsets): same results as the dense layout."""
    ops = _ops()
    _announce("gemm bf16, huge row pitch")
    M, N, K, pitch = 40, 300, 264, (1 << 22) + 8
    a = _rand((M, K), torch.bfloat16, 21)
    b = _rand((N, K), torch.bfloat16, 22)
    big = torch.zeros(M * pitch, dtype=torch.bfloat16, device=DEV)
    av = big.as_strided((M, K), (pitch, 1))
    av.copy_(a.to(DEV))
    out = torch.empty(M, N, dtype=torch.bfloat16, device=DEV)
    ops.gemm(av, b.to(DEV), out)
    dense = torch.empty_like(out)
    ops.gemm(a.to(DEV), b.to(DEV), dense)
    ref = a.float() @ b.float().t()
    assert max_rel_err(out, ref) < TOL[torch.bfloat16] and max_rel_err(dense, ref) < TOL[torch.bfloat16]


def test_empty_inputs_are_no_ops():
    """Zero rows, zero segments, zero tokens: every kernel wrapper returns (an empty result, or its output untouched)
    without a launch error - the shapes an empty rank-local pack or an image-free batch produce."""
    from mi355_vit import ops

    C, H, D = 128, 4, 32
    bf = dict(dtype=torch.bfloat16, device=DEV)
    x0 = torch.empty(0, C, **bf)
    w = torch.ones(C, **bf)
    y, rstd = ops.rmsnorm_fwd(x0, w, 1e-6)
    assert y.shape == (0, C) and rstd.shape == (0,)
    dx, dw = ops.rmsnorm_bwd(x0, x0, w, rstd)
    assert dx.shape == (0, C) and torch.count_nonzero(dw) == 0
    assert ops.colsum(x0, torch.bfloat16).shape == (C,) and torch.count_nonzero(ops.colsum(x0, torch.bfloat16)) == 0
    qkv = torch.empty(0, 3 * H * D, **bf)
    table = torch.empty(0, D, dtype=torch.float32, device=DEV)
    assert ops.rope_(qkv, table, table, 2 * H, D).shape == (0, 3 * H * D)
    assert ops.gather_rows(torch.ones(8, C, **bf), torch.empty(0, dtype=torch.int64, device=DEV)).shape == (0, C)
    dst = torch.full((4, C), 7.0, **bf)
    assert torch.equal(ops.segment_copy(torch.ones(4, C, **bf), dst, []), torch.full((4, C), 7.0, **bf))
    out = torch.full((0, 64), 3.0, **bf)
    ops.gemm(torch.empty(0, C, **bf), torch.ones(64, C, **bf), out)
    q = torch.empty(0, H * D, **bf)
    cu = torch.zeros(1, dtype=torch.int32, device=DEV)
    o, lse = ops.attn_fwd(q, q, q, cu, 0, H, D, D ** -0.5)
    assert o.shape == (0, H * D) and lse.shape == (H, 0)
    dq, dk, dv = (torch.empty_like(q) for _ in range(3))
    ops.attn_bwd(q, q, q, o, o, lse, cu, 0, H, D, D ** -0.5, dq, dk, dv)
    # (a text sequence without image placeholders is an error of its own, as in the reference: test_gpu_handoff.py)
    torch.cuda.synchronize()
