"""CPU restatement of the optimizer step behind ``Trainer.optimizer_step``.

TEST INFRASTRUCTURE ONLY (see ``oracle/__init__.py``).  ``trainer`` below is the
reference file ``python/ray/trainer.py``.

The reference builds ``torch.optim.Adam(params | two weight-decay groups, lr=...,
foreach=False)`` (trainer:479-577), optionally scales every gradient in place by
``min(1, max_norm / (global_norm + 1e-6))`` (trainer:123-156) and calls
``optimizer.step()`` (trainer:158-189).  The arithmetic itself is not in the
reference tree: it is ``torch/optim/adam.py::_single_tensor_adam`` of the
installed torch (2.10; the reference pins no torch version), restated here
operation by operation on plain tensors, with the association and the fused
multiply-adds of torch's CPU kernels (add(alpha), lerp, addcmul, addcdiv).  With
``torch_cpu_quirks=True`` two artefacts of those CPU kernels are reproduced as well
(alpha rounded to bf16 for bf16 tensors; a square root that is not always
correctly rounded) and the results are bit-identical to torch's on the CPU; the
default is plain IEEE arithmetic, which is what the HIP kernel is held to.  Parameters, gradients and both moments
share one dtype; with bf16 every operation rounds its result to bf16, exactly as
the per-tensor torch kernels do (each computes in fp32 and stores bf16).

What pins each function besides its own formula:

========================  ====================================================
``adam_step``             ``torch.optim.Adam(foreach=False)`` itself, run on
                          the CPU for several steps in fp32 and bf16, with and
                          without weight decay (tests/test_oracle_adam.py);
                          closed form for step 1: p1 = p0 - lr * sign(g) (eps -> 0)
``clip_coefficient``      the reference's formula, hand values (trainer:137-138)
``grad_norm_squared``     ``sum(g.double() ** 2)``; equals
                          ``torch.nn.utils.get_total_norm(...) ** 2``
========================  ====================================================
"""

from __future__ import annotations

import math
from typing import Dict, List, Optional, Sequence

import torch


def clip_coefficient(global_norm: float, max_norm: float) -> float:
    """trainer:137-138."""
    return min(1.0, max_norm / (global_norm + 1e-6))


def grad_norm_squared(grads: Sequence[Optional[torch.Tensor]]) -> float:
    """trainer:293-308: sum over tensors of ||g.float()||_2 ** 2, here accumulated in float64."""
    return float(sum(g.detach().double().pow(2).sum().item() for g in grads if g is not None))


def _fma32(a: torch.Tensor, b: torch.Tensor, c: torch.Tensor) -> torch.Tensor:
    """Correctly rounded fp32 fused multiply-add a*b + c of fp32 tensors (one rounding), without an fma routine:
    the product is exact in fp64; the fp64 sum is corrected to round-to-odd with the exact error term of the
    addition (two-sum), after which the final rounding to fp32 cannot double-round (53 >= 24 + 2 bits)."""
    a, b, c = torch.broadcast_tensors(a, b, c)
    prod = a.double() * b.double()
    cd = c.double()
    s = prod + cd
    bv = s - prod  # two-sum: s + err == prod + cd exactly
    err = (prod - (s - bv)) + (cd - bv)
    bits = s.contiguous().view(torch.int64).clone()
    inexact_even = (err != 0) & ((bits & 1) == 0) & torch.isfinite(s)
    toward_larger_magnitude = (err > 0) == (s > 0)
    bits = torch.where(inexact_even, torch.where(toward_larger_magnitude, bits + 1, bits - 1), bits)
    return bits.view(torch.float64).to(torch.float32)


def _r(x: torch.Tensor, dtype: torch.dtype) -> torch.Tensor:
    """Round an fp32 intermediate to the storage dtype and come back to fp32."""
    return x.to(dtype).to(torch.float32)


def adam_step(
    param: torch.Tensor,
    grad: torch.Tensor,
    exp_avg: torch.Tensor,
    exp_avg_sq: torch.Tensor,
    step: int,
    lr: float,
    beta1: float = 0.9,
    beta2: float = 0.999,
    eps: float = 1e-8,
    weight_decay: float = 0.0,
    grad_scale: float = 1.0,
    torch_cpu_quirks: bool = False,
) -> Dict[str, torch.Tensor]:
    """One Adam update of one tensor; ``step`` is the 1-based step count AFTER the increment.

    Returns new ``param``, ``grad`` (scaled when ``grad_scale != 1``), ``exp_avg``, ``exp_avg_sq`` in the input dtype.
    Follows _single_tensor_adam (capturable / differentiable / amsgrad / maximize all off):
      grad = grad.add(param, alpha=weight_decay); exp_avg.lerp_(grad, 1 - beta1);
      exp_avg_sq.mul_(beta2).addcmul_(grad, grad, value=1 - beta2);
      denom = (exp_avg_sq.sqrt() / sqrt(1 - beta2 ** step)).add_(eps);
      param.addcdiv_(exp_avg, denom, value=-(lr / (1 - beta1 ** step)))
    with fma(alpha, param, grad), fma(w, end - start, start), fma(value * g, g, v) and p + (value * m) / denom.
    """
    dt = param.dtype
    f32 = torch.float32
    p, g, m, v = (t.detach().to(f32) for t in (param, grad, exp_avg, exp_avg_sq))
    sc = lambda x: torch.tensor(x, dtype=f32)  # python scalars enter the kernels as fp32
    if grad_scale != 1.0:
        g = _r(g * sc(grad_scale), dt)  # p.grad.mul_(clip_coeff)
    g_out = g
    if weight_decay != 0.0:
        # torch's CPU add kernel converts alpha to the tensors' dtype first (a bf16 0.01 is 0.010009765625); the GPU
        # kernel keeps it in fp32.  The GPU behaviour is the default here; the CPU one is for the pin against torch.
        alpha = sc(weight_decay).to(dt).to(f32) if torch_cpu_quirks else sc(weight_decay)
        g = _r(_fma32(alpha, p, g), dt)  # grad + alpha * param, fused
    w = 1.0 - beta1
    assert abs(w) < 0.5, "lerp's other branch is not restated"
    m = _r(_fma32(sc(w), g - m, m), dt)  # start + weight * (end - start), fused
    v = _r(v * sc(beta2), dt)
    v = _r(_fma32(sc(1.0 - beta2) * g, g, v), dt)  # self + (value * t1) * t2, last product fused
    bias_correction1 = 1.0 - beta1**step
    bias_correction2 = 1.0 - beta2**step
    step_size = lr / bias_correction1
    bias_correction2_sqrt = math.sqrt(bias_correction2)
    # torch's vectorised CPU sqrt is off by one ulp for about 0.7 % of fp32 inputs; the default here is the correctly
    # rounded root (through fp64), the CPU one is for the pin against torch
    d = _r(torch.sqrt(v) if torch_cpu_quirks else torch.sqrt(v.double()).to(f32), dt)
    d = _r(d / sc(bias_correction2_sqrt), dt)
    d = _r(d + sc(eps), dt)
    p = _r(p + (sc(-step_size) * m) / d, dt)  # self + (value * t1) / t2
    return {"param": p.to(dt), "grad": g_out.to(dt), "exp_avg": m.to(dt), "exp_avg_sq": v.to(dt)}


def adam_run(params: List[torch.Tensor], grads_per_step: List[List[torch.Tensor]], lr: float, weight_decay: Sequence[float],
             grad_scale: Optional[Sequence[float]] = None, **kw) -> Dict[str, List[torch.Tensor]]:
    """Several steps over several tensors (zero-initialised moments), for comparisons with an optimizer object."""
    ps = [p.detach().clone() for p in params]
    ms = [torch.zeros_like(p) for p in ps]
    vs = [torch.zeros_like(p) for p in ps]
    for s, grads in enumerate(grads_per_step, start=1):
        gs = 1.0 if grad_scale is None else grad_scale[s - 1]
        for i, g in enumerate(grads):
            out = adam_step(ps[i], g, ms[i], vs[i], s, lr, weight_decay=weight_decay[i], grad_scale=gs, **kw)
            ps[i], ms[i], vs[i] = out["param"], out["exp_avg"], out["exp_avg_sq"]
    return {"param": ps, "exp_avg": ms, "exp_avg_sq": vs}
