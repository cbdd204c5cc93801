"""Tensor-level wrappers over the C ABI.  PyTorch supplies device memory and the current HIP stream;
all arithmetic happens in libmi355vit.so.  Every wrapper validates shapes on the host before a launch."""

from __future__ import annotations

import ctypes as C
import functools
import os as _os
from typing import Optional, Sequence, Tuple

import torch

from . import _lib
from ._lib import BF16, F32, GemmArgs

_DT = {torch.float32: F32, torch.bfloat16: BF16}
N_PARTIAL = 1024  # work-groups (= partial rows) of the RMSNorm backward: 4 per CU keep enough loads in flight

_trace = None  # optional list collecting (tag, info, start_event, end_event) per tagged launch
recomputing = False  # True while a checkpointed block re-runs its forward inside the backward (marks traced launches)


def set_trace(records: Optional[list]) -> None:
    """Give a list to time every tagged kernel launch with a pair of events on the current stream; None stops."""
    global _trace
    _trace = records


_side_streams: dict = {}
OVERLAP_WGRAD = _os.environ.get("MVIT_OVERLAP", "1") != "0"


def side_stream(device: torch.device) -> Optional["torch.cuda.Stream"]:
    """The second stream (default priority) that weight-gradient GEMMs run on so that they fill the idle compute
    units of the input-gradient chain; None while launches are being timed one by one."""
    if not OVERLAP_WGRAD or _trace is not None:
        return None
    key = torch.device(device).index if torch.device(device).index is not None else torch.cuda.current_device()
    st = _side_streams.get(key)
    if st is None:
        st = _side_streams[key] = torch.cuda.Stream(device=key)
    return st


def _launch(tag: str, info: dict, call):
    if _trace is None:
        return call()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    rc = call()
    e1.record()
    _trace.append((tag, dict(info, recompute=recomputing), e0, e1))
    return rc


def dt(t: torch.Tensor) -> int:
    try:
        return _DT[t.dtype]
    except KeyError:
        raise TypeError(f"unsupported dtype {t.dtype} (float32 and bfloat16 only)") from None


# the current stream's handle alone, without building a Stream object per launch (a torch build without the direct
# accessor goes through the object)
_current_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None) or (lambda index: torch.cuda.current_stream(index).cuda_stream)


def _stream(t: torch.Tensor) -> int:
    if not t.is_cuda:
        raise RuntimeError("mi355_vit kernels need tensors on the GPU; there is no CPU path")
    index = t.device.index
    return _current_raw_stream(torch.cuda.current_device() if index is None else index)


def _p(t: Optional[torch.Tensor]) -> Optional[int]:
    return None if t is None else t.data_ptr()


def _rowmajor(t: torch.Tensor, what: str) -> None:
    if t.dim() != 2 or t.stride(1) != 1:
        raise ValueError(f"{what}: expected a 2-D tensor with unit column stride, got shape {tuple(t.shape)} stride {t.stride()}")


# ------------------------------------------------------------------------------ host planners


def rot_pos_ids(grid_thw: torch.Tensor, merge: int) -> torch.Tensor:
    g = grid_thw.detach().to("cpu", torch.int64).contiguous()
    S = int((g[:, 0] * g[:, 1] * g[:, 2]).sum())
    out = torch.empty(S, 2, dtype=torch.int64)
    _lib.check(_lib.load().mvit_rot_pos_ids(g.data_ptr(), g.shape[0], merge, out.data_ptr()), "mvit_rot_pos_ids")
    return out


def window_index(grid_thw: torch.Tensor, merge: int, window_size: int, patch_size: int) -> Tuple[torch.Tensor, torch.Tensor]:
    """Returns (window_index [S/merge^2] int64, cu_window_seqlens int32 without repeated entries), on the CPU."""
    g = grid_thw.detach().to("cpu", torch.int64).contiguous()
    units = int((g[:, 0] * (g[:, 1] // merge) * (g[:, 2] // merge)).sum())
    idx = torch.empty(units, dtype=torch.int64)
    cu = torch.empty(units + 1, dtype=torch.int32)
    n = C.c_int64(0)
    rc = _lib.load().mvit_window_index(g.data_ptr(), g.shape[0], merge, window_size, patch_size, idx.data_ptr(), cu.data_ptr(), cu.numel(), C.addressof(n))
    _lib.check(rc, "mvit_window_index")
    return idx, cu[: n.value].clone()


def cu_seqlens(grid_thw: torch.Tensor) -> torch.Tensor:
    g = grid_thw.detach().to("cpu", torch.int64).contiguous()
    cu = torch.empty(int(g[:, 0].sum()) + 1, dtype=torch.int32)
    n = C.c_int64(0)
    _lib.check(_lib.load().mvit_cu_seqlens(g.data_ptr(), g.shape[0], cu.data_ptr(), cu.numel(), C.addressof(n)), "mvit_cu_seqlens")
    return cu[: n.value]


def sp_token_cuts(sample_len: int, sp: int) -> list:
    out = (C.c_int64 * (sp + 1))()
    _lib.check(_lib.load().mvit_sp_token_cuts(sample_len, sp, C.addressof(out)), "mvit_sp_token_cuts")
    return list(out)


def sp_window_cuts(sample_len: int, sp: int, window_lengths: Sequence[int]) -> Tuple[list, list]:
    n = len(window_lengths)
    wl = (C.c_int64 * max(n, 1))(*window_lengths)
    pos = (C.c_int64 * (sp + 1))()
    idx = (C.c_int64 * (sp + 1))()
    rc = _lib.load().mvit_sp_window_cuts(sample_len, sp, C.addressof(wl) if n else None, n, C.addressof(pos), C.addressof(idx))
    if rc != 0:
        raise ValueError(_lib.load().mvit_last_error().decode())
    return list(pos), list(idx)


# ------------------------------------------------------------------------------ bandwidth kernels


def rmsnorm_fwd(x: torch.Tensor, w: torch.Tensor, eps: float) -> Tuple[torch.Tensor, torch.Tensor]:
    _rowmajor(x, "rmsnorm x")
    if not x.is_contiguous() or w.shape != (x.shape[1],) or w.dtype != x.dtype:
        raise ValueError("rmsnorm_fwd: x must be contiguous [rows, cols] and w [cols] of the same dtype")
    y = torch.empty_like(x)
    rstd = torch.empty(x.shape[0], dtype=torch.float32, device=x.device)
    st = _stream(x)
    rc = _launch("rmsnorm_fwd", {"rows": x.shape[0], "cols": x.shape[1], "esize": x.element_size()},
                 lambda: _lib.load().mvit_rmsnorm_fwd(x.data_ptr(), w.data_ptr(), y.data_ptr(), rstd.data_ptr(), x.shape[0], x.shape[1], eps, dt(x), st))
    _lib.check(rc, "mvit_rmsnorm_fwd")
    return y, rstd


def rmsnorm_bwd(dy, x, w, rstd, dx_add: Optional[torch.Tensor] = None, w_grad_dtype=None):
    """Returns (dx [+ dx_add], dw) in fresh tensors."""
    if not (dy.is_contiguous() and x.is_contiguous()) or dy.shape != x.shape or dy.dtype != x.dtype:
        raise ValueError("rmsnorm_bwd: dy and x must be contiguous with equal shape and dtype")
    if dx_add is not None and (dx_add.shape != x.shape or dx_add.dtype != x.dtype or not dx_add.is_contiguous()):
        raise ValueError("rmsnorm_bwd: dx_add must match x")
    rows, cols = x.shape
    dx = torch.empty_like(x)
    partial = torch.empty(N_PARTIAL, cols, dtype=torch.float32, device=x.device)
    lib = _lib.load()
    st = _stream(x)
    rc = _launch("rmsnorm_bwd", {"rows": rows, "cols": cols, "esize": x.element_size(), "add": dx_add is not None},
                 lambda: lib.mvit_rmsnorm_bwd(dy.data_ptr(), x.data_ptr(), w.data_ptr(), rstd.data_ptr(), _p(dx_add), dx.data_ptr(), partial.data_ptr(), N_PARTIAL, rows, cols, dt(x), st))
    _lib.check(rc, "mvit_rmsnorm_bwd")
    dw = torch.empty(cols, dtype=w_grad_dtype or w.dtype, device=x.device)
    _lib.check(lib.mvit_reduce_partials(partial.data_ptr(), N_PARTIAL, cols, dw.data_ptr(), dt(dw), _stream(x)), "mvit_reduce_partials")
    return dx, dw


def reduce_partials(partial: torch.Tensor, out_dtype: torch.dtype) -> torch.Tensor:
    """Column sums of a contiguous fp32 [n_partial, cols] array of partial sums (fixed order, reproducible)."""
    if partial.dtype != torch.float32 or partial.dim() != 2 or not partial.is_contiguous():
        raise ValueError("reduce_partials: expected a contiguous fp32 2-D tensor")
    out = torch.empty(partial.shape[1], dtype=out_dtype, device=partial.device)
    rc = _lib.load().mvit_reduce_partials(partial.data_ptr(), partial.shape[0], partial.shape[1], out.data_ptr(), dt(out), _stream(partial))
    _lib.check(rc, "mvit_reduce_partials")
    return out


def colsum(x: torch.Tensor, out_dtype: torch.dtype) -> torch.Tensor:
    """Column sums of a 2-D (possibly row-strided) tensor: the bias gradient of a Linear layer."""
    _rowmajor(x, "colsum x")
    rows, cols = x.shape
    npart = max(1, min(64, (rows + 15) // 16))
    partial = torch.empty(npart, cols, dtype=torch.float32, device=x.device)
    lib = _lib.load()
    _lib.check(lib.mvit_colsum(x.data_ptr(), x.stride(0), rows, cols, partial.data_ptr(), npart, dt(x), _stream(x)), "mvit_colsum")
    out = torch.empty(cols, dtype=out_dtype, device=x.device)
    _lib.check(lib.mvit_reduce_partials(partial.data_ptr(), npart, cols, out.data_ptr(), dt(out), _stream(x)), "mvit_reduce_partials")
    return out


def rope_(x: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor, nheads: int, head_dim: int, backward: bool = False,
          lead_heads: int = 0, lead_scale: float = 1.0) -> torch.Tensor:
    """In-place rotary embedding on the first nheads*head_dim columns of each row of x ([rows, >=nheads*head_dim]).
    The first ``lead_heads`` heads are also multiplied by ``lead_scale`` before the one rounding to x's dtype."""
    _rowmajor(x, "rope x")
    rows = x.shape[0]
    for t in (cos, sin):
        if t.dtype != torch.float32 or tuple(t.shape) != (rows, head_dim) or not t.is_contiguous():
            raise ValueError(f"rope: cos/sin must be contiguous fp32 [{rows}, {head_dim}]")
    if x.shape[1] < nheads * head_dim:
        raise ValueError("rope: row narrower than nheads*head_dim")
    if not 0 <= lead_heads <= nheads:
        raise ValueError(f"rope: lead_heads {lead_heads} of {nheads} heads")
    st = _stream(x)
    rc = _launch("rope", {"rows": rows, "nheads": nheads, "head_dim": head_dim, "esize": x.element_size()},
                 lambda: _lib.load().mvit_rope_scaled(x.data_ptr(), cos.data_ptr(), sin.data_ptr(), rows, nheads, head_dim, x.stride(0),
                                                      int(backward), lead_heads, lead_scale, dt(x), st))
    _lib.check(rc, "mvit_rope_scaled")
    return x


def gather_rows(src: torch.Tensor, index: torch.Tensor, rows_per_index: int = 1) -> torch.Tensor:
    """out.view(n, rows_per_index*cols)[i] = src.view(-1, rows_per_index*cols)[index[i]] (bit-exact)."""
    if not src.is_contiguous() or src.dim() != 2:
        raise ValueError("gather_rows: src must be contiguous 2-D")
    if index.dtype != torch.int64 or index.device != src.device or not index.is_contiguous():
        raise ValueError("gather_rows: index must be a contiguous int64 tensor on src's device")
    n_units = src.shape[0] // rows_per_index
    if n_units * rows_per_index != src.shape[0]:
        raise ValueError("gather_rows: rows not divisible by rows_per_index")
    out = torch.empty(index.numel() * rows_per_index, src.shape[1], dtype=src.dtype, device=src.device)
    row_bytes = rows_per_index * src.shape[1] * src.element_size()
    st = _stream(src)
    rc = _launch("gather_rows", {"rows": index.numel(), "row_bytes": row_bytes},
                 lambda: _lib.load().mvit_gather_rows(src.data_ptr(), index.data_ptr(), out.data_ptr(), index.numel(), row_bytes, st))
    _lib.check(rc, "mvit_gather_rows")
    return out


def segment_copy(src: torch.Tensor, dst: torch.Tensor, segments: Sequence[Tuple[int, int, int]]) -> torch.Tensor:
    """Copy rows: for (src_row, dst_row, n_rows) in segments.  Host validates bounds; the kernel moves bytes."""
    if src.dim() != 2 or dst.dim() != 2 or not (src.is_contiguous() and dst.is_contiguous()):
        raise ValueError("segment_copy: src and dst must be contiguous 2-D")
    if src.shape[1] != dst.shape[1] or src.dtype != dst.dtype:
        raise ValueError("segment_copy: column count / dtype mismatch")
    segs = [(int(a), int(b), int(n)) for a, b, n in segments if n > 0]
    for a, b, n in segs:
        if a < 0 or b < 0 or a + n > src.shape[0] or b + n > dst.shape[0]:
            raise ValueError(f"segment_copy: segment ({a},{b},{n}) out of bounds for {src.shape[0]} -> {dst.shape[0]} rows")
    if not segs:
        return dst
    # pinned staging + asynchronous copy: the launch below is ordered behind it on the same stream, the host does not wait
    desc = torch.tensor(segs, dtype=torch.int64).pin_memory().to(src.device, non_blocking=True)
    row_bytes = src.shape[1] * src.element_size()
    rc = _lib.load().mvit_segment_copy(src.data_ptr(), dst.data_ptr(), desc.data_ptr(), len(segs), max(n for _, _, n in segs), row_bytes, _stream(src))
    _lib.check(rc, "mvit_segment_copy")
    return dst


def pad_pack(pack: torch.Tensor, lens: Sequence[int], pad_len: int, pad_value: float) -> Tuple[torch.Tensor, torch.Tensor]:
    if pack.dim() != 2 or not pack.is_contiguous():
        raise ValueError("pad_pack: pack must be contiguous 2-D")
    B = len(lens)
    if sum(lens) != pack.shape[0] or any(n > pad_len for n in lens):
        raise ValueError("pad_pack: lengths do not match the pack or exceed pad_len")
    offs, o = [], 0
    for n in lens:
        offs.append(o)
        o += n
    meta = torch.tensor([list(lens), offs], dtype=torch.int64).pin_memory().to(pack.device, non_blocking=True)
    padded = torch.empty(B, pad_len, pack.shape[1], dtype=pack.dtype, device=pack.device)
    mask = torch.empty(B, pad_len, dtype=torch.uint8, device=pack.device)
    bits = torch.tensor([pad_value], dtype=pack.dtype).view(torch.int16 if pack.element_size() == 2 else torch.int32).item() & (0xFFFF if pack.element_size() == 2 else 0xFFFFFFFF)
    rc = _lib.load().mvit_pad_pack(pack.data_ptr() if pack.numel() else padded.data_ptr(), padded.data_ptr(), mask.data_ptr(), meta[0].data_ptr(), meta[1].data_ptr(), B, pad_len, pack.shape[1], pack.element_size(), bits, _stream(pack))
    _lib.check(rc, "mvit_pad_pack")
    return padded, mask.view(torch.bool)


def cast2d(src: torch.Tensor, dst: torch.Tensor) -> torch.Tensor:
    """dst[:rows, :cols] = cast(src) for row-strided 2-D views."""
    _rowmajor(src, "cast2d src")
    _rowmajor(dst, "cast2d dst")
    if src.shape != dst.shape:
        raise ValueError("cast2d: shape mismatch")
    rc = _lib.load().mvit_cast2d(src.data_ptr(), src.stride(0), dt(src), dst.data_ptr(), dst.stride(0), dt(dst), src.shape[0], src.shape[1], _stream(src))
    _lib.check(rc, "mvit_cast2d")
    return dst


# ------------------------------------------------------------------------------ GEMM


def gemm(
    a: torch.Tensor,
    b: torch.Tensor,
    out: torch.Tensor,
    *,
    trans_a: bool = False,
    trans_b: bool = False,
    epilogue: int = _lib.EPI_NONE,
    bias: Optional[torch.Tensor] = None,
    b2: Optional[torch.Tensor] = None,
    bias2: Optional[torch.Tensor] = None,
    residual: Optional[torch.Tensor] = None,
    aux: Optional[torch.Tensor] = None,
    aux_off: int = 0,
    n: Optional[int] = None,
    split_k: int = 1,
    colsum_partial: Optional[torch.Tensor] = None,
) -> torch.Tensor:
    """out[M, N] = epilogue(A . B^T) with A = a (or a^T if trans_a) and B = b (or b^T if trans_b), see include/mi355_vit.h.

    Shapes: a [M,K] (or [K,M]); b [N,K] (or [K,N]); all 2-D with unit column stride (row strides free).
    ``n`` narrows the logical N (columns of B / out) below b's extent.
    ``colsum_partial`` (EPI_SWIGLU_BWD only): fp32 [ceil(M/256), out.stride(0)] receiving per-tile column sums of out.
    """
    for t, nm in ((a, "a"), (b, "b"), (out, "out")):
        _rowmajor(t, f"gemm {nm}")
    M, K = (a.shape[1], a.shape[0]) if trans_a else (a.shape[0], a.shape[1])
    Nb, Kb = (b.shape[1], b.shape[0]) if trans_b else (b.shape[0], b.shape[1])
    N = Nb if n is None else n
    if Kb != K or N > Nb:
        raise ValueError(f"gemm: contraction mismatch A {tuple(a.shape)} (trans={trans_a}) vs B {tuple(b.shape)} (trans={trans_b})")
    if a.dtype != b.dtype:
        raise ValueError("gemm: A and B dtypes differ")
    width_needed = N + (aux_off if epilogue == _lib.EPI_SWIGLU_BWD else 0)
    if out.shape[0] != M or out.shape[1] < width_needed:
        raise ValueError(f"gemm: out {tuple(out.shape)} too small for M={M}, N={N}")
    args = GemmArgs()
    args.dtype, args.out_dtype = dt(a), dt(out)
    args.trans_a, args.trans_b, args.epilogue = int(trans_a), int(trans_b), epilogue
    args.M, args.N, args.K = M, N, K
    args.A, args.lda = a.data_ptr(), a.stride(0)
    args.B, args.ldb = b.data_ptr(), b.stride(0)
    if b2 is not None:
        _rowmajor(b2, "gemm b2")
        if b2.shape != b.shape or b2.stride(0) != b.stride(0) or b2.dtype != b.dtype:
            raise ValueError("gemm: b2 must match b")
        args.B2 = b2.data_ptr()
    for t, nm in ((bias, "bias"), (bias2, "bias2")):
        if t is not None and (t.dtype != a.dtype or t.numel() < N or not t.is_contiguous()):
            raise ValueError(f"gemm: {nm} must be contiguous, of A's dtype, with at least N entries")
    args.bias, args.bias2 = _p(bias), _p(bias2)
    args.C, args.ldc = out.data_ptr(), out.stride(0)
    if residual is not None:
        _rowmajor(residual, "gemm residual")
        need = N + (aux_off if epilogue == _lib.EPI_SWIGLU_BWD else 0)
        if residual.dtype != a.dtype or residual.shape[0] != M or residual.shape[1] < need:
            raise ValueError("gemm: residual shape/dtype mismatch")
        args.R, args.ldr = residual.data_ptr(), residual.stride(0)
    if aux is not None:
        _rowmajor(aux, "gemm aux")
        need = N + (aux_off if epilogue == _lib.EPI_SWIGLU else 0)
        if aux.dtype != a.dtype or aux.shape[0] != M or aux.shape[1] < need:
            raise ValueError("gemm: aux shape/dtype mismatch")
        args.aux, args.ldaux = aux.data_ptr(), aux.stride(0)
    args.aux_off = aux_off
    if split_k > 1:
        if epilogue not in (_lib.EPI_NONE, _lib.EPI_BIAS, _lib.EPI_BIAS_RES):
            raise ValueError("gemm: split_k needs the plain, the bias or the bias + residual epilogue")
        ws = torch.empty(split_k * M * N, dtype=torch.float32, device=a.device)
        args.workspace, args.workspace_bytes, args.split_k = ws.data_ptr(), ws.numel() * 4, split_k
    if colsum_partial is not None:
        if epilogue != _lib.EPI_SWIGLU_BWD:
            raise ValueError("gemm: colsum_partial is an output of the SwiGLU-backward epilogue only")
        cp = colsum_partial
        if cp.dtype != torch.float32 or not cp.is_contiguous() or cp.shape != (-(-M // 256), out.stride(0)) or cp.device != a.device:
            raise ValueError(f"gemm: colsum_partial must be contiguous fp32 [{-(-M // 256)}, {out.stride(0)}]")
        args.workspace, args.workspace_bytes = cp.data_ptr(), cp.numel() * 4
    st = _stream(a)
    tag = f"gemm_{'t' if trans_a else 'n'}{'t' if trans_b else 'n'}_epi{epilogue}"
    _lib.check(_launch(tag, {"M": M, "N": N, "K": K}, lambda: _lib.load().mvit_gemm(C.byref(args), st)), "mvit_gemm")
    return out


_N_CU = 256  # MI355X compute units; one 256x256 GEMM work-group runs per CU


@functools.lru_cache(maxsize=None)
def wgrad_split_k(out_rows: int, out_cols: int, k: int) -> int:
    """K slices for a GEMM with few output tiles (256x256) and a long contraction: the weight gradients (contraction
    over the tokens).  The model uses it for those only: on a forward or input-gradient GEMM a slice count chosen
    from the batch size would make a row's result depend on how many rows share its batch.

    Picks the slice count with the lowest modelled time.  Work items (tiles x slices) run in rounds of one per
    CU, so the count should fill whole rounds; every slice costs an fp32 partial tile that a second kernel
    re-reads.  Constants are microseconds measured on MI355X (a 32-deep K step takes 0.6 us on a lightly loaded
    chip, 0.95 us when every CU is busy; ~8 us per tile epilogue; ~3.5 TB/s for the partial-sum traffic)."""
    tiles = -(-out_rows // 256) * -(-out_cols // 256)
    best, best_t = 1, None
    for sk in range(1, 17):
        if sk > 1 and k // sk < 512:
            break
        items = tiles * sk
        rounds = -(-items // _N_CU)
        load = items / (rounds * _N_CU)
        steps = -(-(-(-k // sk)) // 64) * 2
        t = rounds * (steps * (0.6 + 0.35 * load) + 8.0)
        if sk > 1:
            t += 5.0 + sk * out_rows * out_cols * 4 / 3.5e6
        if best_t is None or t < best_t:
            best, best_t = sk, t
    return best


# ------------------------------------------------------------------------------ attention


def _attn_view(t: torch.Tensor, nheads: int, head_dim: int, what: str) -> int:
    """t is [S, >= nheads*head_dim] with unit column stride; returns the row stride."""
    _rowmajor(t, what)
    if t.shape[1] < nheads * head_dim:
        raise ValueError(f"{what}: row narrower than nheads*head_dim")
    return t.stride(0)


def segment_order(lengths: torch.Tensor) -> Optional[torch.Tensor]:
    """int32 permutation of the segments, longest first (stable), for the ``seg_order`` argument of the attention
    calls; None when all segments that matter are equally long (the natural order is then as good).  Host tensor in,
    host tensor out."""
    ln = lengths.detach().to("cpu", torch.int64)
    if ln.numel() < 2 or int(ln.max()) <= 64:  # windows: one work-group each, all alike
        return None
    return torch.sort(ln, descending=True, stable=True).indices.to(torch.int32).contiguous()


def check_segments(cu_host: torch.Tensor, total: int, max_seqlen: int, seg_order_host: Optional[torch.Tensor] = None) -> None:
    """Host-side validation of an attention segment list (the kernels trust it): ``cu_host`` (a CPU tensor) must start
    at 0, never decrease and end at ``total``; no segment may be longer than ``max_seqlen`` (rows beyond it would be
    left unwritten); ``seg_order_host`` must be a permutation of the segments.  Raises ValueError."""
    cu = cu_host.detach().to("cpu", torch.int64)
    if cu.dim() != 1 or cu.numel() < 1 or int(cu[0]) != 0:
        raise ValueError("attn: cu_seqlens must be a 1-D list starting at 0")
    lens = cu[1:] - cu[:-1]
    if lens.numel() and int(lens.min()) < 0:
        raise ValueError("attn: cu_seqlens must not decrease")
    if int(cu[-1]) != total:
        raise ValueError(f"attn: cu_seqlens ends at {int(cu[-1])} but the inputs hold {total} rows")
    if lens.numel() and int(lens.max()) > max_seqlen:
        raise ValueError(f"attn: max_seqlen {max_seqlen} is smaller than the longest segment ({int(lens.max())})")
    if seg_order_host is not None:
        o = seg_order_host.detach().to("cpu", torch.int64)
        if o.numel() != lens.numel() or not torch.equal(torch.sort(o).values, torch.arange(lens.numel())):
            raise ValueError("attn: seg_order must be a permutation of the segments")


def _order_ptr(seg_order: Optional[torch.Tensor], cu_seqlens: torch.Tensor) -> Optional[int]:
    if seg_order is None:
        return None
    if seg_order.dtype != torch.int32 or seg_order.device != cu_seqlens.device or not seg_order.is_contiguous() or seg_order.numel() != cu_seqlens.numel() - 1:
        raise ValueError("attn: seg_order must be a contiguous int32 permutation of the segments on the inputs' device")
    return seg_order.data_ptr()


def attn_fwd(q, k, v, cu_seqlens: torch.Tensor, max_seqlen: int, nheads: int, head_dim: int, scale: float, out: Optional[torch.Tensor] = None,
             seg_order: Optional[torch.Tensor] = None):
    """q, k, v: [S, nheads*head_dim] views (row strides free).  Returns (o [S, nheads*head_dim], lse [nheads, S]).
    ``seg_order``: optional scheduling order of the segments (see segment_order); results do not depend on it.
    ``cu_seqlens``, ``max_seqlen`` and ``seg_order`` live on the device and are trusted as they are (checking them
    here would cost a read-back per call): callers validate their host copies once with ``check_segments``."""
    S = q.shape[0]
    if cu_seqlens.dtype != torch.int32 or cu_seqlens.device != q.device or not cu_seqlens.is_contiguous():
        raise ValueError("attn: cu_seqlens must be a contiguous int32 tensor on the inputs' device")
    if k.shape[0] != S or v.shape[0] != S or not (q.dtype == k.dtype == v.dtype):
        raise ValueError("attn: q, k, v row counts / dtypes differ")
    if out is None:
        out = torch.empty(S, nheads * head_dim, dtype=q.dtype, device=q.device)
    lse = torch.empty(nheads, S, dtype=torch.float32, device=q.device)
    order_ptr = _order_ptr(seg_order, cu_seqlens)
    st = _stream(q)
    strides = (_attn_view(q, nheads, head_dim, "attn q"), _attn_view(k, nheads, head_dim, "attn k"),
               _attn_view(v, nheads, head_dim, "attn v"), _attn_view(out, nheads, head_dim, "attn o"))
    rc = _launch("attn_fwd", {"cu": cu_seqlens, "max_seqlen": max_seqlen, "nheads": nheads, "head_dim": head_dim}, lambda: _lib.load().mvit_attn_fwd(
        q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(), lse.data_ptr(), cu_seqlens.data_ptr(), order_ptr,
        cu_seqlens.numel() - 1, max_seqlen, S, nheads, head_dim, *strides, scale, dt(q), st))
    _lib.check(rc, "mvit_attn_fwd")
    return out, lse


def attn_bwd(q, k, v, o, d_o, lse, cu_seqlens, max_seqlen, nheads, head_dim, scale, dq, dk, dv, seg_order: Optional[torch.Tensor] = None):
    """Writes dq, dk, dv ([S, nheads*head_dim] views, row strides free)."""
    order_ptr = _order_ptr(seg_order, cu_seqlens)
    S = q.shape[0]
    for t in (k, v, o, d_o, dq, dk, dv):
        if t.shape[0] != S or t.dtype != q.dtype:
            raise ValueError("attn_bwd: row count / dtype mismatch")
    if tuple(lse.shape) != (nheads, S) or lse.dtype != torch.float32 or not lse.is_contiguous():
        raise ValueError("attn_bwd: lse must be contiguous fp32 [nheads, S]")
    # workspace: delta, and for the long-segment kernels -lse*log2(e) and -delta behind it
    delta = torch.empty(_lib.load().mvit_attn_bwd_delta_elems(max_seqlen, S, nheads, head_dim, dt(q)), dtype=torch.float32, device=q.device)
    st = _stream(q)
    strides = tuple(_attn_view(t, nheads, head_dim, nm) for t, nm in ((q, "q"), (k, "k"), (v, "v"), (o, "o"), (d_o, "do"), (dq, "dq"), (dk, "dk"), (dv, "dv")))
    rc = _launch("attn_bwd", {"cu": cu_seqlens, "max_seqlen": max_seqlen, "nheads": nheads, "head_dim": head_dim}, lambda: _lib.load().mvit_attn_bwd(
        q.data_ptr(), k.data_ptr(), v.data_ptr(), o.data_ptr(), d_o.data_ptr(), lse.data_ptr(),
        dq.data_ptr(), dk.data_ptr(), dv.data_ptr(), delta.data_ptr(), delta.numel(), cu_seqlens.data_ptr(), order_ptr,
        cu_seqlens.numel() - 1, max_seqlen, S, nheads, head_dim, *strides, scale, dt(q), st))
    _lib.check(rc, "mvit_attn_bwd")
    return dq, dk, dv
