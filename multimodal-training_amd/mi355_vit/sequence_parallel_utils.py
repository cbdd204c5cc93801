"""Ragged sequence-parallel pack / unpack on one GPU.

Same function names, arguments and results as the reference's
python/models/qwen2_5_vl/sequence_parallel_utils.py, split in two layers:

* planning (pure host integers, done by the C planners ``mvit_sp_token_cuts`` / ``mvit_sp_window_cuts``)
  produces a ``RaggedSequenceMeta`` -- usable without a GPU;
* data movement (``mvit_segment_copy`` / ``mvit_pad_pack``) turns a plan into one kernel launch instead of
  a Python loop of slices and ``torch.cat``.  Copies are bit-exact.

The collectives of the reference (all-gather / all-to-all) are outside this build; ``gather_rank_packs``
performs the re-interleave that follows the ragged all-gather (modeling_qwen2_5_vl.py:1040-1064) on packs
that are already resident on this GPU.
"""

from __future__ import annotations

import logging
from dataclasses import dataclass
from typing import List, Optional, Sequence, Tuple

import torch

from . import ops

logger = logging.getLogger(__name__)


@dataclass
class RaggedSequenceMeta:
    """Rank-local layout of a ragged pack (field names as in the reference, spu:29-49)."""

    batch_size: int
    local_lengths: List[int]
    global_lengths: List[int]
    sp_rank: int
    sp_size: int
    device: torch.device
    global_sample_offsets: List[int]
    sample_global_slices: List[Tuple[int, int]]
    local_token_offsets: List[Tuple[int, int]]
    window_lengths_per_sample: Optional[List[List[int]]]
    window_index_ranges: Optional[List[Optional[Tuple[int, int]]]]

    def __post_init__(self) -> None:
        self.total_local_len = sum(self.local_lengths)
        self.max_local_len = max(self.local_lengths, default=0)
        self.min_local_len = min(self.local_lengths, default=0)
        self.requires_dummy_pad = self.total_local_len == 0

    def clone_with(self, *, local_lengths=None, sample_global_slices=None, local_token_offsets=None, window_index_ranges=None):
        lens = list(self.local_lengths if local_lengths is None else local_lengths)
        if local_token_offsets is None:
            offs, o = [], 0
            for n in lens:
                offs.append((o, o + n))
                o += n
        else:
            offs = list(local_token_offsets)
        if window_index_ranges is not None:
            wr = list(window_index_ranges)
        else:
            wr = None if self.window_index_ranges is None else list(self.window_index_ranges)
        return RaggedSequenceMeta(
            batch_size=self.batch_size, local_lengths=lens, global_lengths=list(self.global_lengths),
            sp_rank=self.sp_rank, sp_size=self.sp_size, device=self.device,
            global_sample_offsets=list(self.global_sample_offsets),
            sample_global_slices=list(self.sample_global_slices if sample_global_slices is None else sample_global_slices),
            local_token_offsets=offs, window_lengths_per_sample=self.window_lengths_per_sample, window_index_ranges=wr,
        )


def _compute_token_cut_positions(sample_len: int, sp_size: int) -> List[int]:
    return ops.sp_token_cuts(sample_len, sp_size)


def _compute_window_cut_positions(sample_len: int, sp_size: int, window_lengths: Sequence[int]) -> Tuple[List[int], List[int]]:
    return ops.sp_window_cuts(sample_len, sp_size, list(window_lengths))


def _deal_windows(lengths_per_sample: Sequence[int], cu_window_seqlens) -> List[List[int]]:
    cu = [int(v) for v in (cu_window_seqlens.tolist() if torch.is_tensor(cu_window_seqlens) else cu_window_seqlens)]
    wl = [b - a for a, b in zip(cu[:-1], cu[1:])]
    out, cur = [], 0
    for s, n in enumerate(lengths_per_sample):
        got, mine = 0, []
        while got < n and cur < len(wl):
            mine.append(wl[cur])
            got += wl[cur]
            cur += 1
        if got != n:
            raise ValueError(f"Window lengths do not cover sample {s}: {got} vs {n}")
        out.append(mine)
    if cur != len(wl):
        raise ValueError("Unused window lengths remain after per-sample split")
    return out


def plan_split(lengths_per_sample: Sequence[int], sp_rank: int, sp_size: int, cu_window_seqlens=None,
               device: torch.device | str = "cpu") -> RaggedSequenceMeta:
    """Host-only half of split_pack_by_sp: which global rows does `sp_rank` own?"""
    lengths = [int(n) for n in lengths_per_sample]
    windows = _deal_windows(lengths, cu_window_seqlens) if cu_window_seqlens is not None else None
    local, slices, local_offs, wranges, goffs = [], [], [], [], []
    g = lo = 0
    for s, n in enumerate(lengths):
        goffs.append(g)
        if windows is not None:
            cuts, idxs = _compute_window_cut_positions(n, sp_size, windows[s])
            if sp_rank == 0 and any(a == b for a, b in zip(cuts[:-1], cuts[1:])):
                logger.warning(
                    "Sequence parallel requested %d chunks but sample %d only provides %d window(s) (%d tokens). "
                    "Some ranks will receive empty slices; consider increasing `data.min_pixels`/`data.max_pixels` "
                    "or reducing the sequence parallel degree.", sp_size, s, len(windows[s]), n)
            wranges.append((idxs[sp_rank], idxs[sp_rank + 1]))
        else:
            cuts = _compute_token_cut_positions(n, sp_size)
        a, b = cuts[sp_rank], cuts[sp_rank + 1]
        local.append(b - a)
        slices.append((g + a, g + b))
        local_offs.append((lo, lo + b - a))
        lo += b - a
        g += n
    return RaggedSequenceMeta(
        batch_size=len(lengths), local_lengths=local, global_lengths=lengths, sp_rank=sp_rank, sp_size=sp_size,
        device=torch.device(device), global_sample_offsets=goffs, sample_global_slices=slices,
        local_token_offsets=local_offs, window_lengths_per_sample=windows,
        window_index_ranges=wranges if windows is not None else None,
    )


def split_pack_by_sp(tokens: torch.Tensor, lengths_per_sample: Sequence[int], sp_rank: int, sp_size: int,
                     cu_window_seqlens: Optional[torch.Tensor] = None, debug: bool = False):
    """Rows of the global pack owned by `sp_rank`, concatenated in sample order, plus their layout."""
    meta = plan_split(lengths_per_sample, sp_rank, sp_size, cu_window_seqlens, tokens.device)
    out = torch.empty(meta.total_local_len, tokens.shape[-1], dtype=tokens.dtype, device=tokens.device)
    segs = [(a, lo, b - a) for (a, b), (lo, _) in zip(meta.sample_global_slices, meta.local_token_offsets)]
    ops.segment_copy(tokens.contiguous(), out, segs)
    if debug:
        logger.info("[Rank %d] split_pack_by_sp: global=%d -> local=%d, local_lens=%s", sp_rank, tokens.shape[0], out.shape[0], meta.local_lengths)
    return out, meta


def pad_pack_to_batch(pack_rank: torch.Tensor, meta: RaggedSequenceMeta, pad_value: float = 0.0,
                      pad_to: Optional[int] = None, enforce_min_pad: int = 0):
    want = meta.max_local_len if pad_to is None else pad_to
    if want < meta.max_local_len:
        raise ValueError(f"Requested pad length {want} < local max {meta.max_local_len}")
    return ops.pad_pack(pack_rank.contiguous(), meta.local_lengths, max(want, enforce_min_pad), pad_value)


def unpad_batch_to_pack(padded: torch.Tensor, mask: torch.Tensor, *, return_lengths: bool = False):
    B, L, Hd = padded.shape
    lengths = mask.sum(dim=1).tolist()  # host sync, as in the reference (spu:340)
    out = torch.empty(sum(lengths), Hd, dtype=padded.dtype, device=padded.device)
    segs, o = [], 0
    for b, n in enumerate(lengths):
        segs.append((b * L, o, n))
        o += n
    ops.segment_copy(padded.contiguous().view(B * L, Hd), out, segs)
    return out, (lengths if return_lengths else None)


def rebuild_local_cu_seqlens(meta: RaggedSequenceMeta, *, use_windows: bool = False) -> torch.Tensor:
    if not use_windows:
        cu, t = [0], 0
        for n in meta.local_lengths:
            t += n
            cu.append(t)
        return torch.tensor(cu, device=meta.device, dtype=torch.int32)
    if meta.window_lengths_per_sample is None or meta.window_index_ranges is None:
        raise ValueError("Window metadata not available in RaggedSequenceMeta")
    cu, t = [0], 0
    for wl, rng in zip(meta.window_lengths_per_sample, meta.window_index_ranges):
        if rng is None:
            continue
        for n in wl[rng[0] : rng[1]]:
            t += n
            cu.append(t)
    return torch.tensor(cu, device=meta.device, dtype=torch.int32)


def build_local_rope(meta: RaggedSequenceMeta, global_pos_emb_cos: torch.Tensor, global_pos_emb_sin: torch.Tensor,
                     pad_to: Optional[int] = None):
    segs = [(a, lo, b - a) for (a, b), (lo, _) in zip(meta.sample_global_slices, meta.local_token_offsets)]
    outs = []
    for src in (global_pos_emb_cos, global_pos_emb_sin):
        dst = torch.empty(meta.total_local_len, src.shape[-1], dtype=src.dtype, device=src.device)
        outs.append(ops.segment_copy(src.contiguous(), dst, segs))
    if pad_to is None:
        return outs[0], outs[1], None
    cos_p, mask = ops.pad_pack(outs[0], meta.local_lengths, pad_to, 0.0)
    sin_p, _ = ops.pad_pack(outs[1], meta.local_lengths, pad_to, 0.0)
    return cos_p, sin_p, mask


def gather_rank_packs(rank_packs: Sequence[torch.Tensor], lengths_matrix: Sequence[Sequence[int]]) -> torch.Tensor:
    """Rebuild per-sample order from every rank's pack; lengths_matrix[r][s] = rows of sample s on rank r."""
    sp, B = len(rank_packs), len(lengths_matrix[0]) if lengths_matrix else 0
    ref = rank_packs[0]
    out = torch.empty(sum(int(p.shape[0]) for p in rank_packs), ref.shape[-1], dtype=ref.dtype, device=ref.device)
    segs = [[] for _ in range(sp)]  # per source pack: (row in that pack, row in the output, count)
    cursor, o = [0] * sp, 0
    for s in range(B):
        for r in range(sp):
            n = int(lengths_matrix[r][s])
            if n:
                segs[r].append((cursor[r], o, n))
                cursor[r] += n
                o += n
    for r, pack in enumerate(rank_packs):
        ops.segment_copy(pack.contiguous(), out, segs[r])
    return out


def compute_max_length_across_ranks(local_max_len: int, group=None) -> int:
    """One process, one GPU: the maximum over ranks is the local value (the reference all-reduces, spu:448-459)."""
    return local_max_len
