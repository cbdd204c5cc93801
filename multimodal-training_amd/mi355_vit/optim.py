"""Multi-tensor optimizer step and gradient norm on the GPU.

``FusedAdam`` is ``torch.optim.Adam(..., foreach=False)`` — the optimizer the reference builds in
python/ray/trainer.py:479-577 and steps in trainer.py:158-189 — with the same constructor arguments, parameter
groups, per-parameter state (``step``, ``exp_avg``, ``exp_avg_sq``) and therefore the same ``state_dict``; only
``step()`` differs: one kernel launch over all parameters instead of about ten launches per parameter, with the
clipping coefficient of ``Trainer._clip_gradients`` (trainer.py:123-156) applied inside the same pass.
``grad_norm_squared`` replaces the per-tensor ``norm(2).item() ** 2`` loop of trainer.py:293-308 by two
launches and one read-back.

There is no CPU path: parameters must live on the GPU and the HIP library must be built.
"""

from __future__ import annotations

import ctypes as C
import math
import os
from typing import Dict, Iterable, List, Optional, Tuple

import numpy as np
import torch

from . import _lib

_TABLE_DTYPE = np.dtype(
    [("param", "<u8"), ("grad", "<u8"), ("exp_avg", "<u8"), ("exp_avg_sq", "<u8"), ("numel", "<i8"), ("first_chunk", "<i8"),
     ("step_size", "<f4"), ("bias_correction2_sqrt", "<f4"), ("weight_decay", "<f4"), ("unused", "<f4"),
     ("shadow", "<u8"), ("shadow_cols", "<i8"), ("shadow_ld", "<i8"), ("shadow_dtype", "<i4"), ("unused2", "<i4")]
)
assert _TABLE_DTYPE.itemsize == C.sizeof(_lib.AdamTensor) == 96
_NO_SHADOW = (0, 0, 0, 0, 0)


def attach_shadow(param: torch.Tensor, copy: torch.Tensor) -> None:
    """Declare ``copy`` (a 1-D or 2-D view with unit column stride, of the parameter's dtype or bfloat16) the operand
    copy of ``param`` that the kernels read: ``FusedAdam.step`` then stores every updated element there as well, so
    the copy never has to be rebuilt after a step.  ``copy`` must have the parameter's shape."""
    if copy.shape != param.shape or copy.dim() not in (1, 2) or copy.stride(-1) != 1 or copy.device != param.device:
        raise ValueError("attach_shadow: the copy must be a 1-D / 2-D unit-stride view of the parameter's shape on its device")
    if copy.dtype not in (param.dtype, torch.bfloat16):
        raise ValueError("attach_shadow: the copy's dtype must be the parameter's or bfloat16")
    global _SHADOW_GENERATION
    param._mvit_shadow = copy
    _SHADOW_GENERATION += 1  # every plan built before this call is stale


_SHADOW_GENERATION = 0


def check_shadows(params) -> None:
    """Debug aid (``MVIT_CHECK_SHADOWS=1`` runs it before every step): every operand copy must equal its parameter,
    cast to the copy's dtype.  A writer that updates parameters through raw pointers without storing the copy too
    (another fused optimizer, a custom kernel) leaves the copies stale with no version bump; this is what finds it."""
    for p in params:
        sh = getattr(p, "_mvit_shadow", None)
        if sh is not None and not torch.equal(sh, p.detach().to(sh.dtype)):
            raise RuntimeError(f"operand copy of a parameter of shape {tuple(p.shape)} differs from the parameter: something updated it "
                               "through a raw pointer without storing the copy (see attach_shadow)")


def _shadow_fields(p: torch.Tensor) -> tuple:
    sh = getattr(p, "_mvit_shadow", None)
    if sh is None:
        return _NO_SHADOW
    cols = sh.shape[-1]
    ld = sh.stride(0) if sh.dim() == 2 else cols
    return (sh.data_ptr(), cols, ld, _dtype_code(sh.dtype), 0)


def _check_tensor(t: torch.Tensor, what: str) -> None:
    if not t.is_cuda:
        raise RuntimeError(f"{what}: tensor on {t.device}; the multi-tensor kernels need GPU tensors (there is no CPU path)")
    if t.is_sparse or t.is_complex() or not t.is_contiguous():
        raise RuntimeError(f"{what}: dense, real, contiguous tensors only (got shape {tuple(t.shape)}, stride {t.stride()})")


def _dtype_code(dtype: torch.dtype) -> int:
    if dtype == torch.float32:
        return _lib.F32
    if dtype == torch.bfloat16:
        return _lib.BF16
    raise TypeError(f"unsupported dtype {dtype} (float32 and bfloat16 only)")


def _upload(table: np.ndarray, device: torch.device) -> torch.Tensor:
    # a plain (synchronous) host-to-device copy of a few tens of KB: the table is rebuilt every step because
    # gradients are new allocations after zero_grad(set_to_none=True)
    return torch.from_numpy(table.view(np.uint8)).to(device)


class _Bucket:
    """The tensors of one launch (same device, dtype, betas, eps) with everything that does not change between
    steps: parameter / moment addresses, sizes, chunk starts.  Gradient addresses and the step-dependent scalars
    are filled in per step."""

    def __init__(self, device, dtype, beta1, beta2, eps):
        self.device, self.dtype, self.beta1, self.beta2, self.eps = device, dtype, beta1, beta2, eps
        self.params: List[torch.Tensor] = []
        self.step_tensors: List[torch.Tensor] = []
        self.rows: List[tuple] = []
        self.group_slices: List[Tuple[int, int, int]] = []  # (group index, first row, end row)

    def finish(self) -> None:
        self.table, self.n_chunks = _build_table(self.rows)
        self.steps = np.array([int(t.item()) for t in self.step_tensors], dtype=np.int64)


class FusedAdam(torch.optim.Adam):
    """Adam with the arithmetic of torch's single-tensor path, stepped by one multi-tensor launch per dtype."""

    def __init__(self, params, lr: float = 1e-3, betas: Tuple[float, float] = (0.9, 0.999), eps: float = 1e-8,
                 weight_decay: float = 0.0, *, foreach: Optional[bool] = False):
        if foreach:
            raise ValueError("FusedAdam replaces the foreach=False optimizer of the reference; foreach must stay False")
        super().__init__(params, lr=lr, betas=betas, eps=eps, weight_decay=weight_decay, foreach=False)
        self._plan_key: Optional[tuple] = None
        self._plan: List[_Bucket] = []

    def load_state_dict(self, state_dict) -> None:
        super().load_state_dict(state_dict)
        self._plan_key = None  # moments and step counts were replaced

    def _init_state(self, p: torch.Tensor) -> dict:
        st = self.state[p]
        if len(st) == 0:  # same entries and dtypes as torch.optim.Adam (capturable and fused off)
            st["step"] = torch.tensor(0.0, dtype=torch.float32)
            st["exp_avg"] = torch.zeros_like(p, memory_format=torch.preserve_format)
            st["exp_avg_sq"] = torch.zeros_like(p, memory_format=torch.preserve_format)
        return st

    def _make_plan(self) -> List[_Bucket]:
        buckets: Dict[tuple, _Bucket] = {}
        for gi, group in enumerate(self.param_groups):
            if any(group.get(k) for k in ("amsgrad", "maximize", "capturable", "differentiable", "decoupled_weight_decay")):
                raise RuntimeError("FusedAdam: amsgrad / maximize / capturable / differentiable / decoupled_weight_decay are not built")
            beta1, beta2 = group["betas"]
            touched = []
            for p in group["params"]:
                if p.grad is None:
                    continue
                _check_tensor(p, "FusedAdam parameter")
                st = self._init_state(p)
                m, v = st["exp_avg"], st["exp_avg_sq"]
                _check_tensor(m, "FusedAdam exp_avg")
                _check_tensor(v, "FusedAdam exp_avg_sq")
                if m.dtype != p.dtype or v.dtype != p.dtype or m.shape != p.shape or v.shape != p.shape:
                    raise RuntimeError("FusedAdam: optimizer state dtype / shape differs from its parameter")
                if p.numel() == 0:
                    continue
                key = (p.device, p.dtype, beta1, beta2, group["eps"])
                bk = buckets.get(key)
                if bk is None:
                    bk = buckets[key] = _Bucket(*key)
                if bk not in touched:
                    touched.append(bk)
                    bk.group_slices.append([gi, len(bk.rows), len(bk.rows)])
                bk.params.append(p)
                bk.step_tensors.append(st["step"])
                bk.rows.append((p.data_ptr(), 0, m.data_ptr(), v.data_ptr(), p.numel(), 0, 0.0, 0.0, 0.0, 0.0) + _shadow_fields(p))
                bk.group_slices[-1][2] = len(bk.rows)
        for bk in buckets.values():
            bk.finish()
        return list(buckets.values())

    @torch.no_grad()
    def step(self, closure=None, grad_scale: float = 1.0, write_grad: bool = True):
        """One optimizer step.  ``grad_scale`` multiplies every gradient first (the clipping coefficient); with
        ``write_grad`` the scaled gradients are stored back, as the reference's in-place scaling leaves them."""
        loss = None
        if closure is not None:
            with torch.enable_grad():
                loss = closure()
        # which parameters take part (those with a gradient) and where they and their moments live rarely changes:
        # the table is rebuilt only when it does; per step only gradient addresses and scalars are refreshed
        key = (_SHADOW_GENERATION, tuple((id(p), p.data_ptr()) for group in self.param_groups for p in group["params"] if p.grad is not None))
        if os.environ.get("MVIT_CHECK_SHADOWS") == "1":
            check_shadows(p for group in self.param_groups for p in group["params"])
        stale = key != self._plan_key or any(
            int(bk.step_tensors[0].item()) != int(bk.steps[0]) or int(bk.step_tensors[-1].item()) != int(bk.steps[-1])
            for bk in self._plan)  # step counters edited from outside (cheap spot check of the host mirror)
        if stale:
            self._plan = self._make_plan()
            self._plan_key = key
        lib = _lib.load()
        for bk in self._plan:
            n = len(bk.params)
            grads = [p.grad for p in bk.params]
            for p, g in zip(bk.params, grads):
                if not g.is_cuda or not g.is_contiguous() or g.dtype != bk.dtype or g.shape != p.shape:
                    _check_tensor(g, "FusedAdam gradient")
                    raise RuntimeError("FusedAdam: gradient dtype / shape differs from its parameter")
            table = bk.table
            table["grad"][:n] = [g.data_ptr() for g in grads]
            torch._foreach_add_(bk.step_tensors, 1.0)
            bk.steps += 1
            for gi, lo, hi in bk.group_slices:
                group = self.param_groups[gi]
                lr = float(group["lr"])
                table["weight_decay"][lo:hi] = group["weight_decay"]
                steps = bk.steps[lo:hi]
                for step in np.unique(steps).tolist():  # one value unless some tensors joined later
                    rows = lo + np.nonzero(steps == step)[0]
                    table["step_size"][rows] = lr / (1.0 - bk.beta1**step)  # python floats, as torch/optim/adam.py
                    table["bias_correction2_sqrt"][rows] = math.sqrt(1.0 - bk.beta2**step)
            dev_table = _upload(table, bk.device)
            with torch.cuda.device(bk.device):
                stream = torch.cuda.current_stream(bk.device).cuda_stream
                rc = lib.mvit_adam_step(dev_table.data_ptr(), n, bk.n_chunks, bk.beta1, bk.beta2, bk.eps, float(grad_scale),
                                        int(bool(write_grad)), _dtype_code(bk.dtype), stream)
            _lib.check(rc, "mvit_adam_step")
        return loss


def _build_table(rows: List[tuple]) -> Tuple[np.ndarray, int]:
    """Rows (in _TABLE_DTYPE field order, first_chunk ignored) -> host table with chunk starts and the sentinel."""
    n = len(rows)
    table = np.zeros(n + 1, dtype=_TABLE_DTYPE)
    cols = list(zip(*rows))
    for name, col in zip(_TABLE_DTYPE.names, cols):
        if name != "first_chunk":
            table[name][:n] = col
    counts = -(-table["numel"][:n] // _lib.ADAM_CHUNK)
    table["first_chunk"][1:] = np.cumsum(counts)
    return table, int(table["first_chunk"][n])


def grad_norm_squared(params: Iterable[torch.Tensor], static_scratch: bool = False) -> float:
    """sum over parameters of ||grad||_2^2 (fp32 within a chunk of 8192 elements, fp64 across chunks): the quantity
    Trainer._compute_grad_norm_squared returns, with one host read-back in total.  ``static_scratch`` keeps the
    per-chunk partial sums in the array built into the library (mvit_grad_sumsq_static) instead of a fresh tensor."""
    buckets: Dict[tuple, List[tuple]] = {}
    for p in params:
        g = p.grad
        if g is None or g.numel() == 0:
            continue
        _check_tensor(g, "grad_norm_squared gradient")
        buckets.setdefault((g.device, g.dtype), []).append((0, g.data_ptr(), 0, 0, g.numel(), 0, 0.0, 0.0, 0.0, 0.0) + _NO_SHADOW)
    lib = _lib.load()
    outs = []
    for (device, dtype), rows in buckets.items():
        table, n_chunks = _build_table(rows)
        dev_table = _upload(table, device)
        out = torch.empty(1, dtype=torch.float64, device=device)
        with torch.cuda.device(device):
            stream = torch.cuda.current_stream(device).cuda_stream
            if static_scratch:
                rc = lib.mvit_grad_sumsq_static(dev_table.data_ptr(), len(rows), n_chunks, out.data_ptr(), _dtype_code(dtype), stream)
            else:
                partial = torch.empty(n_chunks, dtype=torch.float32, device=device)
                rc = lib.mvit_grad_sumsq(dev_table.data_ptr(), len(rows), n_chunks, partial.data_ptr(), out.data_ptr(),
                                         _dtype_code(dtype), stream)
        _lib.check(rc, "mvit_grad_sumsq")
        outs.append(out)
    if not outs:
        return 0.0
    total = outs[0] if len(outs) == 1 else torch.stack([o.to(outs[0].device) for o in outs]).sum(0)
    return float(total.item())
