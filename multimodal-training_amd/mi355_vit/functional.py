"""Autograd functions of the vision tower.  Each one is a fixed sequence of C-ABI kernel launches with a
hand-written backward (no autograd graph inside), so a transformer block is one node of PyTorch's graph.

Reference spans (python/models/qwen2_5_vl/modeling_qwen2_5_vl.py):
  VisionBlockFn   Qwen2_5_VLVisionBlock.forward :776-792 with _forward_standard :385-472 and the MLP :203-204
  PatchEmbedFn    Qwen2_5_VisionPatchEmbed.forward :225-231
  PermuteRowsFn   window reorder :934-937 and its inverse :1067-1068
  MergerFn        Qwen2_5_VLPatchMerger.forward :260-262
"""

from __future__ import annotations

import ctypes
import os
from dataclasses import dataclass
from typing import Dict, List, Optional, Tuple

import torch

from . import _lib, ops

E = _lib


def round_up(v: int, m: int) -> int:
    return (v + m - 1) // m * m


@dataclass
class BlockWeights:
    """Compute-dtype operands of one block, laid out for the fused GEMMs.

    wqkv [3C, C] / bqkv [3C]         q, k, v stacked
    wgu  [2*Ipad, C] / bgu [2*Ipad]  gate rows [0, I), up rows [Ipad, Ipad+I); padding rows are zero
    wdown [C, Ipad] / bdown [C]      padding columns are zero
    """

    norm1: torch.Tensor
    norm2: torch.Tensor
    wqkv: torch.Tensor
    bqkv: torch.Tensor
    wproj: torch.Tensor
    bproj: torch.Tensor
    wgu: torch.Tensor
    bgu: torch.Tensor
    wdown: torch.Tensor
    bdown: torch.Tensor
    C: int
    I: int
    Ipad: int
    alias: bool = False  # norm1 / norm2 / wproj / bproj / bdown are the parameters themselves (same dtype), not copies


# order of the parameter tensors handed to VisionBlockFn
LOG2E = 1.4426950408889634  # log2(e): the attention kernels work in base-2 exponentials

BLOCK_PARAM_ORDER = (
    "norm1.weight", "norm2.weight",
    "attn.q_proj.weight", "attn.q_proj.bias", "attn.k_proj.weight", "attn.k_proj.bias",
    "attn.v_proj.weight", "attn.v_proj.bias", "attn.proj.weight", "attn.proj.bias",
    "mlp.gate_proj.weight", "mlp.gate_proj.bias", "mlp.up_proj.weight", "mlp.up_proj.bias",
    "mlp.down_proj.weight", "mlp.down_proj.bias",
)


def pack_block_weights(params: List[torch.Tensor], dtype: torch.dtype, into: Optional[BlockWeights]) -> BlockWeights:
    """(Re)fill the packed operands from the 16 parameters (cast to `dtype` on the way).

    Operands that are a single parameter (norm weights, proj, the down bias) are the parameter itself when it
    already has the compute dtype; the fused ones (q|k|v, gate|up, the padded down weight) are copies.  Every copy is
    declared to the optimizer (``optim.attach_shadow``): ``FusedAdam.step`` writes updated values into it directly, so
    an optimizer step never forces a re-pack; any other in-place change of a parameter bumps its version counter and
    the owner of the pack calls this function again."""
    from .optim import attach_shadow

    (n1, n2, wq, bq, wk, bk, wv, bv, wp, bp, wg, bg, wu, bu, wd, bd) = params
    C = wq.shape[1]
    I = wg.shape[0]
    Ipad = round_up(I, 8)
    dev = wq.device
    alias = all(p.dtype == dtype and p.is_contiguous() for p in (n1, n2, wp, bp, bd))
    if into is None or into.wqkv.dtype != dtype or into.wqkv.device != dev or into.alias != alias:
        z = lambda *s: torch.zeros(*s, dtype=dtype, device=dev)  # noqa: E731
        e = (lambda *s: None) if alias else z  # noqa: E731
        into = BlockWeights(e(1, C), e(1, C), z(3 * C, C), z(1, 3 * C), e(C, C), e(1, C), z(2 * Ipad, C), z(1, 2 * Ipad),
                            z(C, Ipad), e(1, C), C, I, Ipad, alias)
    cp = ops.cast2d
    v = lambda t: t.detach().view(1, -1)  # noqa: E731

    def fill(param: torch.Tensor, dst: torch.Tensor) -> None:
        cp(param.detach() if param.dim() == 2 else v(param), dst)
        attach_shadow(param, dst if param.dim() == 2 else dst.view(-1))

    if alias:
        into.norm1, into.norm2, into.wproj, into.bproj, into.bdown = v(n1), v(n2), wp.detach(), v(bp), v(bd)
        for param in (n1, n2, wp, bp, bd):
            param._mvit_shadow = None  # read in place: nothing to keep in step
    else:
        for param, dst in ((n1, into.norm1), (n2, into.norm2), (wp, into.wproj), (bp, into.bproj), (bd, into.bdown)):
            fill(param, dst)
    for j, (w, b) in enumerate(((wq, bq), (wk, bk), (wv, bv))):
        fill(w, into.wqkv[j * C : (j + 1) * C])
        fill(b, into.bqkv[:, j * C : (j + 1) * C])
    for j, (w, b) in enumerate(((wg, bg), (wu, bu))):
        fill(w, into.wgu[j * Ipad : j * Ipad + I])
        fill(b, into.bgu[:, j * Ipad : j * Ipad + I])
    fill(wd, into.wdown[:, :I])
    return into


@dataclass
class AttnGeometry:
    """Per-layer attention layout: device cu_seqlens, the longest segment, head counts, rotary tables."""

    cu: torch.Tensor
    max_seqlen: int
    nheads: int
    head_dim: int
    cos: torch.Tensor  # fp32 [S, head_dim]
    sin: torch.Tensor
    order: Optional[torch.Tensor] = None  # device int32 permutation of the segments, longest first (ops.segment_order)


# One C call per block and direction (mvit_block_fwd / mvit_block_bwd) instead of one per kernel: the same launches with
# the same operands, issued from inside the library.  MVIT_BLOCK_CALLS=0 keeps the call-by-call sequence below, which is
# also what runs while launches are being timed one by one (ops.set_trace) and for parameters of mixed gradient dtypes.
BLOCK_CALLS = os.environ.get("MVIT_BLOCK_CALLS", "1") != "0"
_join_events: dict = {}


def _block_args(x: torch.Tensor, W: BlockWeights, geo: AttnGeometry, eps: float) -> "_lib.BlockArgs":
    a = _lib.BlockArgs()
    a.dtype = ops.dt(x)
    a.S, a.C, a.I, a.Ipad, a.nheads, a.head_dim = x.shape[0], W.C, W.I, W.Ipad, geo.nheads, geo.head_dim
    a.eps, a.q_lead_scale, a.attn_scale = eps, geo.head_dim**-0.5 * LOG2E, 1.0 / LOG2E
    a.n_seg, a.max_seqlen = geo.cu.numel() - 1, geo.max_seqlen
    a.norm1, a.norm2, a.wqkv, a.bqkv, a.wproj = W.norm1.data_ptr(), W.norm2.data_ptr(), W.wqkv.data_ptr(), W.bqkv.data_ptr(), W.wproj.data_ptr()
    a.bproj, a.wgu, a.bgu, a.wdown, a.bdown = W.bproj.data_ptr(), W.wgu.data_ptr(), W.bgu.data_ptr(), W.wdown.data_ptr(), W.bdown.data_ptr()
    a.cu, a.cos, a.sin = geo.cu.data_ptr(), geo.cos.data_ptr(), geo.sin.data_ptr()
    a.seg_order = None if geo.order is None else geo.order.data_ptr()
    a.x = x.data_ptr()
    return a


def _block_geometry_ok(x: torch.Tensor, W: BlockWeights, geo: AttnGeometry) -> bool:
    """What the call-by-call wrappers check launch by launch, once for the block: operand layouts the C sequence assumes."""
    S, hd = x.shape[0], geo.head_dim
    return (x.is_cuda and x.is_contiguous() and x.shape[1] == W.C and geo.nheads * hd == W.C
            and geo.cu.dtype == torch.int32 and geo.cu.is_contiguous() and geo.cu.device == x.device
            and all(t.dtype == torch.float32 and tuple(t.shape) == (S, hd) and t.is_contiguous() for t in (geo.cos, geo.sin))
            and (geo.order is None or (geo.order.dtype == torch.int32 and geo.order.is_contiguous() and geo.order.numel() == geo.cu.numel() - 1))
            and all(t.is_contiguous() and t.dtype == x.dtype for t in (W.norm1, W.norm2, W.wqkv, W.bqkv, W.wproj, W.bproj, W.wgu, W.bgu, W.wdown, W.bdown)))


def _block_forward_one_call(x, W, geo, eps, attn_out, for_backward, output):
    S, C = x.shape
    dev, T = x.device, x.dtype
    f32 = torch.float32
    n1, x1, n2 = torch.empty_like(x), torch.empty_like(x), torch.empty_like(x)
    rstd1, rstd2 = torch.empty(S, dtype=f32, device=dev), torch.empty(S, dtype=f32, device=dev)
    qkv = torch.empty(S, 3 * C, dtype=T, device=dev)
    if attn_out is None:
        o, lse = torch.empty_like(x), torch.empty(geo.nheads, S, dtype=f32, device=dev)
    else:
        o, lse = attn_out
    gu = torch.empty(S, 2 * W.Ipad, dtype=T, device=dev) if for_backward else None
    h = torch.empty(S, W.Ipad, dtype=T, device=dev)
    x2 = torch.empty_like(x) if output else None
    a = _block_args(x, W, geo, eps)
    a.skip_attention = int(attn_out is not None)
    a.n1, a.qkv, a.o, a.x1, a.n2, a.h = n1.data_ptr(), qkv.data_ptr(), o.data_ptr(), x1.data_ptr(), n2.data_ptr(), h.data_ptr()
    a.rstd1, a.rstd2, a.lse = rstd1.data_ptr(), rstd2.data_ptr(), lse.data_ptr()
    a.gu, a.x2 = ops._p(gu), ops._p(x2)
    _lib.check(_lib.load().mvit_block_fwd(ctypes.byref(a), ops._stream(x)), "mvit_block_fwd")
    return x2, (rstd1, n1, qkv, o, lse, x1, rstd2, n2, gu, h)


def _block_backward_one_call(dx2, x, saved, W, geo, gdt):
    rstd1, n1, qkv, o, lse, x1, rstd2, n2, gu, h = saved
    S, Cc = x.shape
    I, Ipad = W.I, W.Ipad
    dev, T = x.device, x.dtype
    G = gdt["norm1.weight"]
    e = lambda *shape, dtype=T: torch.empty(*shape, dtype=dtype, device=dev)  # noqa: E731
    dx, dn, dx1 = torch.empty_like(x), torch.empty_like(x), torch.empty_like(x)
    dgu, dqkv = e(S, 2 * Ipad), e(S, 3 * Cc)
    g_n1, g_n2, g_bp, g_bd = e(Cc, dtype=G), e(Cc, dtype=G), e(Cc, dtype=G), e(Cc, dtype=G)
    g_wqkv, g_bqkv = e(3 * Cc, Cc, dtype=G), e(3 * Cc, dtype=G)
    g_wp, g_wgu, g_bgu, g_wd = e(Cc, Cc, dtype=G), e(2 * Ipad, Cc, dtype=G), e(2 * Ipad, dtype=G), e(Cc, I, dtype=G)
    a = _block_args(x, W, geo, 0.0)
    a.grad_dtype = ops._DT[G]
    a.n1, a.qkv, a.o, a.x1, a.n2, a.gu, a.h = n1.data_ptr(), qkv.data_ptr(), o.data_ptr(), x1.data_ptr(), n2.data_ptr(), gu.data_ptr(), h.data_ptr()
    a.rstd1, a.rstd2, a.lse = rstd1.data_ptr(), rstd2.data_ptr(), lse.data_ptr()
    a.dx2, a.dx, a.dgu, a.dn, a.dx1, a.dqkv = dx2.data_ptr(), dx.data_ptr(), dgu.data_ptr(), dn.data_ptr(), dx1.data_ptr(), dqkv.data_ptr()
    a.g_norm1, a.g_norm2, a.g_wqkv, a.g_bqkv, a.g_wproj = g_n1.data_ptr(), g_n2.data_ptr(), g_wqkv.data_ptr(), g_bqkv.data_ptr(), g_wp.data_ptr()
    a.g_bproj, a.g_wgu, a.g_bgu, a.g_wdown, a.g_bdown = g_bp.data_ptr(), g_wgu.data_ptr(), g_bgu.data_ptr(), g_wd.data_ptr(), g_bd.data_ptr()
    sk = ops.wgrad_split_k
    a.split_k_down, a.split_k_gate_up, a.split_k_proj, a.split_k_qkv = sk(Cc, I, S), sk(2 * Ipad, Cc, S), sk(Cc, Cc, S), sk(3 * Cc, Cc, S)
    side = ops.side_stream(dev)
    if side is not None:
        key = dev.index if dev.index is not None else torch.cuda.current_device()
        evs = _join_events.get(key)
        if evs is None:
            evs = [torch.cuda.Event() for _ in range(5)]
            for ev in evs:
                ev.record()  # an event object gets its handle with its first record
            _join_events[key] = evs
        a.side_stream = side.cuda_stream
        for i, ev in enumerate(evs):
            a.events[i] = ev.cuda_event
    lib = _lib.load()
    nbytes = lib.mvit_block_bwd_workspace_bytes(ctypes.byref(a))
    ws = torch.empty(nbytes, dtype=torch.uint8, device=dev)
    a.workspace, a.workspace_bytes = ws.data_ptr(), nbytes
    _lib.check(lib.mvit_block_bwd(ctypes.byref(a), ops._stream(x)), "mvit_block_bwd")
    grads = (
        g_n1, g_n2,
        g_wqkv[:Cc], g_bqkv[:Cc], g_wqkv[Cc : 2 * Cc], g_bqkv[Cc : 2 * Cc], g_wqkv[2 * Cc :], g_bqkv[2 * Cc :],
        g_wp, g_bp,
        g_wgu[:I], g_bgu[:I], g_wgu[Ipad : Ipad + I], g_bgu[Ipad : Ipad + I],
        g_wd, g_bd,
    )
    return dx, grads


def _block_forward(x: torch.Tensor, W: BlockWeights, geo: AttnGeometry, eps: float,
                   attn_out: Optional[Tuple[torch.Tensor, torch.Tensor]] = None, *,
                   for_backward: bool = True, output: bool = True) -> Tuple[Optional[torch.Tensor], tuple]:
    """``attn_out`` = (o, lse) kept from an earlier run of the same block on the same input: the attention product is
    then not computed again (the recomputation of a checkpointed block).

    ``for_backward=False``: nothing but the block's output (and the attention output) will be used, so the gate / up
    pre-activations are not written (the first run of a checkpointed block).  ``output=False``: the block's output is
    not wanted, so the down projection is skipped (the re-run of a checkpointed block: the backward reads `h`, not
    `x2`)."""
    if BLOCK_CALLS and ops._trace is None and _block_geometry_ok(x, W, geo):
        return _block_forward_one_call(x, W, geo, eps, attn_out, for_backward, output)
    S, C = x.shape
    H, hd = geo.nheads, geo.head_dim
    n1, rstd1 = ops.rmsnorm_fwd(x, W.norm1.view(-1), eps)
    qkv = torch.empty(S, 3 * C, dtype=x.dtype, device=x.device)
    ops.gemm(n1, W.wqkv, qkv, epilogue=E.EPI_BIAS, bias=W.bqkv.view(-1))
    # q and k are the first 2*H heads of every row.  The queries leave the rotary pass multiplied by the softmax scale
    # in base-2 units (Q_SCALE), in the same fp32 -> storage rounding as the rotation; the attention kernels then get
    # scale = 1 / log2(e), for which their own pre-scaling of the queries is the identity.  Scores are computed from
    # operands rounded once, as in the reference (the kernels alone would round q * scale a second time).
    ops.rope_(qkv, geo.cos, geo.sin, 2 * H, hd, lead_heads=H, lead_scale=hd**-0.5 * LOG2E)
    if attn_out is None:
        o, lse = ops.attn_fwd(qkv[:, :C], qkv[:, C : 2 * C], qkv[:, 2 * C :], geo.cu, geo.max_seqlen, H, hd, 1.0 / LOG2E,
                              seg_order=geo.order)
    else:
        o, lse = attn_out
    x1 = torch.empty_like(x)
    ops.gemm(o, W.wproj, x1, epilogue=E.EPI_BIAS_RES, bias=W.bproj.view(-1), residual=x)
    n2, rstd2 = ops.rmsnorm_fwd(x1, W.norm2.view(-1), eps)
    gu = torch.empty(S, 2 * W.Ipad, dtype=x.dtype, device=x.device) if for_backward else None
    h = torch.empty(S, W.Ipad, dtype=x.dtype, device=x.device)
    bgu = W.bgu.view(-1)
    ops.gemm(n2, W.wgu[: W.Ipad], h, epilogue=E.EPI_SWIGLU, b2=W.wgu[W.Ipad :], bias=bgu[: W.Ipad], bias2=bgu[W.Ipad :],
             aux=gu, aux_off=W.Ipad)
    x2 = None
    if output:
        x2 = torch.empty_like(x)
        ops.gemm(h, W.wdown, x2, epilogue=E.EPI_BIAS_RES, bias=W.bdown.view(-1), residual=x1)
    return x2, (rstd1, n1, qkv, o, lse, x1, rstd2, n2, gu, h)


def _block_backward(dx2: torch.Tensor, x: torch.Tensor, saved: tuple, W: BlockWeights, geo: AttnGeometry, gdt: Dict[str, torch.dtype]):
    """Returns (dx, grads in BLOCK_PARAM_ORDER).  gdt maps parameter name -> gradient dtype."""
    rstd1, n1, qkv, o, lse, x1, rstd2, n2, gu, h = saved
    S, C = x.shape
    H, hd = geo.nheads, geo.head_dim
    I, Ipad = W.I, W.Ipad
    dev = x.device
    dx2 = dx2.contiguous()
    if (BLOCK_CALLS and ops._trace is None and len(set(gdt.values())) == 1 and gdt["norm1.weight"] in ops._DT and dx2.dtype == x.dtype
            and _block_geometry_ok(x, W, geo)):
        return _block_backward_one_call(dx2, x, saved, W, geo, gdt)
    main = torch.cuda.current_stream(dev)
    side = ops.side_stream(dev)

    def off_chain(fn):
        # work that feeds nothing else in this block (weight and bias gradients) runs on the second stream, after
        # the point its inputs are complete on the main stream, and is joined before the gradients are handed back;
        # one event and one stream switch per point serve the bias and the weight gradient that start there
        if side is None:
            return fn()
        ev = torch.cuda.Event()
        ev.record(main)
        with torch.cuda.stream(side):
            side.wait_event(ev)
            return fn()

    def wgrad(dy, act, out, **kw):
        ops.gemm(dy, act, out, trans_a=True, trans_b=True, split_k=ops.wgrad_split_k(out.shape[0], out.shape[1], S), **kw)

    # ---- MLP: x2 = x1 + down(silu(g) * u)
    g_wd = torch.empty(C, I, dtype=gdt["mlp.down_proj.weight"], device=dev)
    g_bd = off_chain(lambda: (ops.colsum(dx2, gdt["mlp.down_proj.bias"]), wgrad(dx2, h, g_wd, n=I))[0])
    dgu = torch.empty(S, 2 * Ipad, dtype=x.dtype, device=dev)
    # the epilogue also hands back per-tile column sums of dgu: the gate / up bias gradient without re-reading dgu
    part = torch.empty(-(-S // 256), 2 * Ipad, dtype=torch.float32, device=dev)
    ops.gemm(dx2, W.wdown, dgu, trans_b=True, epilogue=E.EPI_SWIGLU_BWD, residual=gu, aux_off=Ipad, colsum_partial=part)
    g_wgu = torch.empty(2 * Ipad, C, dtype=gdt["mlp.gate_proj.weight"], device=dev)
    g_bgu = off_chain(lambda: (ops.reduce_partials(part, gdt["mlp.gate_proj.bias"]), wgrad(dgu, n2, g_wgu))[0])
    dn2 = torch.empty_like(x)
    ops.gemm(dgu, W.wgu, dn2, trans_b=True)
    dx1, g_n2 = ops.rmsnorm_bwd(dn2, x1, W.norm2.view(-1), rstd2, dx_add=dx2, w_grad_dtype=gdt["norm2.weight"])

    # ---- attention: x1 = x + proj(attn(rope(qkv(norm1(x)))))
    g_wp = torch.empty(C, C, dtype=gdt["attn.proj.weight"], device=dev)
    g_bp = off_chain(lambda: (ops.colsum(dx1, gdt["attn.proj.bias"]), wgrad(dx1, o, g_wp))[0])
    d_o = dn2  # reuse the buffer
    ops.gemm(dx1, W.wproj, d_o, trans_b=True)
    dqkv = torch.empty_like(qkv)
    ops.attn_bwd(qkv[:, :C], qkv[:, C : 2 * C], qkv[:, 2 * C :], o, d_o, lse, geo.cu, geo.max_seqlen, H, hd, 1.0 / LOG2E,
                 dqkv[:, :C], dqkv[:, C : 2 * C], dqkv[:, 2 * C :], seg_order=geo.order)
    # dq arrives as the gradient with respect to the scaled, rotated queries: the same factor on the way back
    ops.rope_(dqkv, geo.cos, geo.sin, 2 * H, hd, backward=True, lead_heads=H, lead_scale=hd**-0.5 * LOG2E)
    g_wqkv = torch.empty(3 * C, C, dtype=gdt["attn.q_proj.weight"], device=dev)
    g_bqkv = off_chain(lambda: (ops.colsum(dqkv, gdt["attn.q_proj.bias"]), wgrad(dqkv, n1, g_wqkv))[0])
    dn1 = d_o
    ops.gemm(dqkv, W.wqkv, dn1, trans_b=True)
    dx, g_n1 = ops.rmsnorm_bwd(dn1, x, W.norm1.view(-1), rstd1, dx_add=dx1, w_grad_dtype=gdt["norm1.weight"])
    if side is not None:
        main.wait_stream(side)

    grads = (
        g_n1, g_n2,
        g_wqkv[:C], g_bqkv[:C], g_wqkv[C : 2 * C], g_bqkv[C : 2 * C], g_wqkv[2 * C :], g_bqkv[2 * C :],
        g_wp, g_bp,
        g_wgu[:I], g_bgu[:I], g_wgu[Ipad : Ipad + I], g_bgu[Ipad : Ipad + I],
        g_wd, g_bd,
    )
    return dx, grads


KEEP_ATTENTION_ABOVE = 64  # segments longer than this (the full-attention layers) keep their attention output when checkpointed


class VisionBlockFn(torch.autograd.Function):
    """One transformer block.  With `checkpoint` only the block input is kept and the forward is re-run in
    the backward (the native counterpart of torch.utils.checkpoint around the block, [tf] modeling_layers.py:79).
    A full-attention layer also keeps its attention output and log-sum-exp ([S, C] + [H, S] fp32: 164 MiB at 65,536
    patches), so the re-run skips the one product whose cost grows with the square of the segment length; the values
    it would recompute are bit-identical, hence so are the gradients."""

    @staticmethod
    def forward(ctx, x, holder, geo: AttnGeometry, eps: float, checkpoint: bool, *params):
        W = holder.packed(x.dtype)
        x = x.contiguous()
        differentiated = any(ctx.needs_input_grad)  # False under torch.no_grad() and for frozen inputs and weights
        x2, saved = _block_forward(x, W, geo, eps, for_backward=differentiated and not checkpoint)
        if not differentiated:
            return x2
        ctx.holder, ctx.geo, ctx.eps, ctx.checkpoint = holder, geo, eps, checkpoint
        ctx.gdt = {name: p.dtype for name, p in zip(BLOCK_PARAM_ORDER, params)}
        ctx.x = x
        ctx.saved = None if checkpoint else saved
        ctx.attn_out = (saved[3], saved[4]) if checkpoint and geo.max_seqlen > KEEP_ATTENTION_ABOVE else None
        return x2

    @staticmethod
    def backward(ctx, dx2):
        x, geo = ctx.x, ctx.geo
        W = ctx.holder.packed(x.dtype)
        saved = ctx.saved
        if saved is None:
            ops.recomputing = True
            try:
                _, saved = _block_forward(x, W, geo, ctx.eps, ctx.attn_out, output=False)
            finally:
                ops.recomputing = False
        dx, grads = _block_backward(dx2, x, saved, W, geo, ctx.gdt)
        ctx.saved = None
        ctx.x = None
        ctx.attn_out = None
        return (dx, None, None, None, None) + tuple(grads)


class PatchEmbedFn(torch.autograd.Function):
    """[S, 1176] pixels x Conv3d weight viewed as [C, 1176]: a GEMM without bias."""

    @staticmethod
    def forward(ctx, pixels, weight, compute_dtype):
        w2 = weight.detach().reshape(weight.shape[0], -1)
        K = w2.shape[1]
        px = pixels.detach().reshape(-1, K)
        if px.dtype != compute_dtype or not px.is_contiguous():
            px = ops.cast2d(px if px.stride(1) == 1 else px.contiguous(), torch.empty(px.shape, dtype=compute_dtype, device=px.device))
        if w2.dtype != compute_dtype:
            w2 = ops.cast2d(w2, torch.empty(w2.shape, dtype=compute_dtype, device=w2.device))
        out = torch.empty(px.shape[0], w2.shape[0], dtype=compute_dtype, device=px.device)
        ops.gemm(px, w2, out)
        ctx.px, ctx.wshape, ctx.wdtype = px, weight.shape, weight.dtype
        return out

    @staticmethod
    def backward(ctx, dout):
        px = ctx.px
        gw = torch.empty(dout.shape[1], px.shape[1], dtype=ctx.wdtype, device=px.device)
        ops.gemm(dout.contiguous(), px, gw, trans_a=True, trans_b=True, split_k=ops.wgrad_split_k(gw.shape[0], gw.shape[1], px.shape[0]))
        return None, gw.view(ctx.wshape), None


class PatchEmbedFramesFn(torch.autograd.Function):
    """The patch embedding straight from decoded uint8 frames (bf16 compute): the forward makes the rows of
    ``pixel_values`` inside the GEMM and never writes them; the weight gradient needs them as a matrix, so the backward
    writes them once (``patchify``) just before its GEMM and drops them again."""

    @staticmethod
    def forward(ctx, weight, out_dtype, *frames):
        from . import pixels

        out, _ = pixels.patch_embed_frames(frames, pixels.pack_patch_embed_weight(weight), dtype=out_dtype)
        ctx.frames, ctx.wshape, ctx.wdtype = frames, weight.shape, weight.dtype
        return out

    @staticmethod
    def backward(ctx, dout):
        from . import pixels

        px, _ = pixels.patchify(ctx.frames, dtype=torch.bfloat16)
        dy = dout.contiguous()
        if dy.dtype != torch.bfloat16:
            dy = ops.cast2d(dy, torch.empty(dy.shape, dtype=torch.bfloat16, device=dy.device))
        gw = torch.empty(dy.shape[1], px.shape[1], dtype=ctx.wdtype, device=px.device)
        ops.gemm(dy, px, gw, trans_a=True, trans_b=True, split_k=ops.wgrad_split_k(gw.shape[0], gw.shape[1], px.shape[0]))
        return (gw.view(ctx.wshape), None) + (None,) * len(ctx.frames)


class PermuteRowsFn(torch.autograd.Function):
    """out.view(n, unit*cols)[i] = x.view(n, unit*cols)[index[i]]; `inverse` is the inverse permutation."""

    @staticmethod
    def forward(ctx, x, index, inverse, unit):
        ctx.inverse, ctx.unit = inverse, unit
        return ops.gather_rows(x.contiguous(), index, unit)

    @staticmethod
    def backward(ctx, dout):
        return ops.gather_rows(dout.contiguous(), ctx.inverse, ctx.unit), None, None, None


def _as_dtype(t: torch.Tensor, dtype: torch.dtype) -> torch.Tensor:
    t = t.detach()
    if t.dtype == dtype and t.is_contiguous():
        return t
    t2 = t.reshape(1, -1) if t.dim() == 1 else t
    out = ops.cast2d(t2.contiguous() if t2.stride(-1) != 1 else t2, torch.empty(t2.shape, dtype=dtype, device=t.device))
    return out.view(t.shape)


class MergerFn(torch.autograd.Function):
    """RMSNorm(C) -> view [S/unit, unit*C] -> Linear + exact GELU -> Linear."""

    @staticmethod
    def forward(ctx, x, ln_w, w0, b0, w2, b2, unit, eps):
        T = x.dtype
        x = x.contiguous()
        lw, W0, B0, W2, B2 = (_as_dtype(t, T) for t in (ln_w, w0, b0, w2, b2))
        ln, rstd = ops.rmsnorm_fwd(x, lw, eps)
        M = x.shape[0] // unit
        ln2 = ln.view(M, -1)
        z = torch.empty(M, W0.shape[0], dtype=T, device=x.device)
        y1 = torch.empty_like(z)
        ops.gemm(ln2, W0, y1, epilogue=E.EPI_BIAS_GELU, bias=B0, aux=z)
        y2 = torch.empty(M, W2.shape[0], dtype=T, device=x.device)
        ops.gemm(y1, W2, y2, epilogue=E.EPI_BIAS, bias=B2)
        ctx.saved = (x, lw, rstd, ln2, z, y1, W0, W2)
        ctx.gdt = (ln_w.dtype, w0.dtype, b0.dtype, w2.dtype, b2.dtype)
        return y2

    @staticmethod
    def backward(ctx, dy):
        x, lw, rstd, ln2, z, y1, W0, W2 = ctx.saved
        ctx.saved = None
        dy = dy.contiguous()
        dev = x.device
        g_b2 = ops.colsum(dy, ctx.gdt[4])
        g_w2 = torch.empty(W2.shape, dtype=ctx.gdt[3], device=dev)
        ops.gemm(dy, y1, g_w2, trans_a=True, trans_b=True, split_k=ops.wgrad_split_k(g_w2.shape[0], g_w2.shape[1], dy.shape[0]))
        dz = torch.empty_like(z)
        ops.gemm(dy, W2, dz, trans_b=True, epilogue=E.EPI_GELU_BWD, residual=z)
        g_b0 = ops.colsum(dz, ctx.gdt[2])
        g_w0 = torch.empty(W0.shape, dtype=ctx.gdt[1], device=dev)
        ops.gemm(dz, ln2, g_w0, trans_a=True, trans_b=True, split_k=ops.wgrad_split_k(g_w0.shape[0], g_w0.shape[1], dz.shape[0]))
        dln = torch.empty_like(ln2)
        ops.gemm(dz, W0, dln, trans_b=True)
        dx, g_ln = ops.rmsnorm_bwd(dln.view(x.shape), x, lw, rstd, w_grad_dtype=ctx.gdt[0])
        return dx, g_ln, g_w0, g_b0, g_w2, g_b2, None, None
