"""Pure-Python / numpy restatement of the ragged sequence-parallel index arithmetic.

TEST INFRASTRUCTURE ONLY (see ``oracle/__init__.py``).  ``spu`` below is the
reference file ``python/models/qwen2_5_vl/sequence_parallel_utils.py``;
``modeling`` is ``python/models/qwen2_5_vl/modeling_qwen2_5_vl.py``.

Every function here is integer work and must agree bit-for-bit with the
product.  What pins each one besides its own formula:

========================  ====================================================
``token_cuts``            reference known answers [8,12]/2, [7,11]/3, [100]/4,
                          [2]/4 (tests/test_sequence_parallel_ragged.py:66-137)
``window_cuts``           known answers: windows [6,4]+[7,7] sp2 -> [0,6,13]
                          (:226-243); one window / 4 ranks -> {0,0,0,5}
                          (:331-361); brute-force invariants for sp in 1..8
``split_slices``          the same known answers (exact slices :86-89)
``pad_rows``/``unpad``    round trip, mask layout, pad value -999 (:143-201)
``local_cu``              [4,7,2] -> [0,4,11,13] (:207-224)
``local_rope_slices``     slices [0:6] and [12:16] for [12,8]/2 rank 0 (:249-273)
``reinterleave``          split -> concat-by-rank -> reinterleave is the
                          identity (tests/test_split_gather.py:37-223 semantics)
========================  ====================================================
"""

from __future__ import annotations

from bisect import bisect_left
from typing import List, Optional, Sequence, Tuple

import numpy as np


def token_cuts(n: int, sp: int) -> List[int]:
    """spu:105-114 -- the first ``n % sp`` ranks get one extra token."""
    q, r = divmod(n, sp)
    return [k * q + min(k, r) for k in range(sp + 1)]


def window_cuts(n: int, sp: int, windows: Sequence[int]) -> Tuple[List[int], List[int]]:
    """spu:117-164 -- cut at window boundaries nearest (from above) to k*n/sp.

    Returns (token positions, window indices), both of length sp+1.  The index
    chosen for step k is ``bisect_left(prefix, n*k//sp)`` searched from the
    previous cut, then clamped to ``len(prefix) - (sp - k)`` (but never below the
    previous cut, never negative, never past the last prefix entry).
    """
    if not windows:
        raise ValueError("Window-based splitting requested but no window lengths were provided.")
    if any(w <= 0 for w in windows):
        raise ValueError("non-positive window length")
    prefix = np.concatenate([[0], np.cumsum(np.asarray(windows, dtype=np.int64))]).tolist()
    if prefix[-1] != n:
        raise ValueError(f"Window lengths do not sum to sample length: {prefix[-1]} vs expected {n}")
    idxs = [0]
    for k in range(1, sp):
        prev = idxs[-1]
        i = max(bisect_left(prefix, (n * k) // sp, lo=prev), prev)
        cap = min(max(len(prefix) - (sp - k), prev, 0), len(prefix) - 1)
        idxs.append(min(i, cap, len(prefix) - 1))
    idxs.append(len(prefix) - 1)
    return [prefix[i] for i in idxs], idxs


def windows_per_sample(lengths: Sequence[int], cu_window: Sequence[int]) -> List[List[int]]:
    """spu:186-203 -- deal consecutive window lengths to samples until each is covered."""
    wl = np.diff(np.asarray(cu_window, dtype=np.int64)).tolist()
    out, cur = [], 0
    for s, n in enumerate(lengths):
        got, mine = 0, []
        while got < n and cur < len(wl):
            mine.append(int(wl[cur]))
            got += int(wl[cur])
            cur += 1
        if got != n:
            raise ValueError(f"Window lengths do not cover sample {s}: {got} vs {n}")
        out.append(mine)
    if cur != len(wl):
        raise ValueError("Unused window lengths remain after per-sample split")
    return out


def split_slices(lengths: Sequence[int], rank: int, sp: int, cu_window: Optional[Sequence[int]] = None):
    """spu:167-283 -- per-sample global [start, end) owned by ``rank`` (+ window index ranges)."""
    wins = windows_per_sample(lengths, cu_window) if cu_window is not None else None
    slices, wranges, off = [], [], 0
    for s, n in enumerate(lengths):
        if wins is not None:
            cuts, idxs = window_cuts(n, sp, wins[s])
            wranges.append((idxs[rank], idxs[rank + 1]))
        else:
            cuts = token_cuts(n, sp)
        slices.append((off + cuts[rank], off + cuts[rank + 1]))
        off += n
    return slices, (wranges if wins is not None else None), wins


def split_rows(x: np.ndarray, lengths, rank, sp, cu_window=None) -> np.ndarray:
    """Rows of ``x`` this rank holds, concatenated in sample order (spu:265-269)."""
    slices, _, _ = split_slices(lengths, rank, sp, cu_window)
    parts = [x[a:b] for a, b in slices if b > a]
    return np.concatenate(parts, axis=0) if parts else x[:0]


def pad_rows(pack: np.ndarray, local_lengths: Sequence[int], pad_value=0.0, pad_to=None, enforce_min_pad=0):
    """spu:300-327."""
    mx = max(local_lengths) if len(local_lengths) else 0
    want = mx if pad_to is None else pad_to
    if want < mx:
        raise ValueError(f"Requested pad length {want} < local max {mx}")
    L = max(want, enforce_min_pad)
    out = np.full((len(local_lengths), L) + pack.shape[1:], pad_value, dtype=pack.dtype)
    mask = np.zeros((len(local_lengths), L), dtype=bool)
    off = 0
    for b, n in enumerate(local_lengths):
        out[b, :n] = pack[off : off + n]
        mask[b, :n] = True
        off += n
    return out, mask


def unpad(padded: np.ndarray, mask: np.ndarray):
    """spu:330-350 -- the first ``mask.sum(1)`` rows of every sample."""
    lens = mask.sum(axis=1).tolist()
    parts = [padded[b, :n] for b, n in enumerate(lens) if n > 0]
    pack = np.concatenate(parts, axis=0) if parts else padded.reshape((-1,) + padded.shape[2:])[:0]
    return pack, lens


def local_cu(local_lengths: Sequence[int]) -> np.ndarray:
    """spu:362-368."""
    return np.concatenate([[0], np.cumsum(np.asarray(local_lengths, dtype=np.int64))]).astype(np.int32)


def local_window_cu(wins: List[List[int]], wranges: List[Tuple[int, int]]) -> np.ndarray:
    """spu:370-384."""
    cu, tot = [0], 0
    for w, (a, b) in zip(wins, wranges):
        for n in w[a:b]:
            tot += n
            cu.append(tot)
    return np.asarray(cu, dtype=np.int32)


def reinterleave(rank_packs: List[np.ndarray], lengths_matrix: np.ndarray) -> np.ndarray:
    """modeling:1040-1064 -- rebuild per-sample order from the per-rank packs.

    ``lengths_matrix[r, s]`` = rows of sample ``s`` held by rank ``r``.
    """
    offs = [0] * len(rank_packs)
    parts = []
    for s in range(lengths_matrix.shape[1]):
        for r, pack in enumerate(rank_packs):
            n = int(lengths_matrix[r, s])
            if n:
                parts.append(pack[offs[r] : offs[r] + n])
                offs[r] += n
    return np.concatenate(parts, axis=0) if parts else rank_packs[0][:0]
