"""Pins oracle/adam_oracle.py against torch.optim.Adam(foreach=False) on the CPU: the optimizer the reference
builds (python/ray/trainer.py:479-577) and steps (trainer.py:158-189), and against closed forms."""

import math

import pytest
import torch

from oracle import adam_oracle


def _torch_adam_run(params, grads_per_step, lr, wds, grad_scale=None):
    ps = [torch.nn.Parameter(p.detach().clone()) for p in params]
    groups = [{"params": [p], "weight_decay": wd} for p, wd in zip(ps, wds)]
    opt = torch.optim.Adam(groups, lr=lr, foreach=False)
    for s, grads in enumerate(grads_per_step):
        for p, g in zip(ps, grads):
            p.grad = g.detach().clone()
            if grad_scale is not None and grad_scale[s] != 1.0:
                p.grad.data.mul_(grad_scale[s])  # Trainer._clip_gradients
        opt.step()
    return {"param": [p.detach() for p in ps], "exp_avg": [opt.state[p]["exp_avg"] for p in ps],
            "exp_avg_sq": [opt.state[p]["exp_avg_sq"] for p in ps]}


def _case(dtype, seed, steps=4, aligned=False):
    g = torch.Generator().manual_seed(seed)
    shapes = [(32, 22), (1280,), (4, 16, 3), (64,)] if aligned else [(37, 19), (1280,), (5, 7, 3), (1,)]
    params = [(torch.randn(s, generator=g) * 0.05).to(dtype) for s in shapes]
    grads = [[(torch.randn(s, generator=g) * 10.0 ** float(torch.randint(-4, 1, (1,), generator=g))).to(dtype) for s in shapes] for _ in range(steps)]
    return params, grads


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("wd", [0.0, 0.01])
@pytest.mark.parametrize("seed", [0, 1])
def test_oracle_matches_torch_adam(dtype, wd, seed):
    """Bit-identical parameters and moments after four steps with clipping on two of them.

    bf16 with weight decay uses tensor sizes that are multiples of 64: torch's CPU add(alpha) kernel rounds the
    product alpha * param to bf16 in its scalar tail loop but not in its vector body, so its result for an element
    depends on where the element sits in the tensor; the oracle restates the vector body."""
    params, grads = _case(dtype, seed, aligned=(dtype == torch.bfloat16 and wd != 0.0))
    wds = [wd, 0.0, wd, wd]
    scale = [1.0, 0.37, 1.0, 0.5]
    ref = _torch_adam_run(params, grads, 1e-3, wds, scale)
    got = adam_oracle.adam_run(params, grads, 1e-3, wds, scale, torch_cpu_quirks=True)
    for key in ("param", "exp_avg", "exp_avg_sq"):
        for a, b in zip(got[key], ref[key]):
            assert a.dtype == b.dtype == dtype
            assert torch.equal(a, b), (key, (a.float() - b.float()).abs().max().item())
    # without the two artefacts of torch's CPU kernels (see the oracle) the moments stay identical in fp32 and the
    # parameters move by at most one unit in the last place on a small fraction of the entries
    plain = adam_oracle.adam_run(params, grads, 1e-3, wds, scale)
    for key in ("param", "exp_avg", "exp_avg_sq"):
        for a, b in zip(plain[key], ref[key]):
            a, b = a.float(), b.float()
            if dtype == torch.float32 and key != "param":
                assert torch.equal(a, b), key
            ulp = torch.maximum(a.abs(), b.abs()) * (2.0**-23 if dtype == torch.float32 else 2.0**-8)
            assert bool(((a - b).abs() <= 4 * ulp + 1e-30).all()), key
            assert (a != b).float().mean().item() <= 0.05, key


def test_fma_emulation_is_correctly_rounded():
    """_fma32 against exact rational arithmetic on values chosen to sit near rounding ties."""
    from fractions import Fraction

    g = torch.Generator().manual_seed(5)
    a = torch.randn(400, generator=g)
    b = torch.randn(400, generator=g)
    c = -(a.double() * b.double()).float() + torch.randn(400, generator=g) * 1e-7  # heavy cancellation
    c[:50] = 1.0
    a[:50] = 1.0 + 2.0**-12
    b[:50] = 1.0 + 2.0**-12 + torch.arange(50) * 2.0**-23  # products land on / near half-ulp points
    got = adam_oracle._fma32(a, b, c)
    for i in range(400):
        exact = Fraction(a[i].item()) * Fraction(b[i].item()) + Fraction(c[i].item())
        lo = torch.tensor(float(exact), dtype=torch.float64)  # nearest fp64, then pick the nearer fp32 neighbour exactly
        cand = lo.float()
        nxt = torch.nextafter(cand, torch.tensor(float("inf") if Fraction(cand.item()) < exact else float("-inf")))
        d0, d1 = abs(Fraction(cand.item()) - exact), abs(Fraction(nxt.item()) - exact)
        if d1 < d0:
            best = nxt
        elif d1 == d0:  # tie: even mantissa
            best = cand if (cand.view(torch.int32).item() & 1) == 0 else nxt
        else:
            best = cand
        assert got[i].item() == best.item(), i


def test_first_step_closed_form():
    """Step 1 from zero moments: m = (1-b1) g, v = (1-b2) g^2, both bias corrections cancel, so
    p1 = p0 - lr * g / (|g| + eps)."""
    g = torch.Generator().manual_seed(3)
    p = torch.randn(1000, generator=g)
    gr = torch.randn(1000, generator=g)
    out = adam_oracle.adam_step(p, gr, torch.zeros_like(p), torch.zeros_like(p), 1, 1e-2)
    expect = p - 1e-2 * gr / (gr.abs() + 1e-8)
    assert torch.allclose(out["param"], expect, rtol=1e-5, atol=1e-7)
    assert torch.allclose(out["exp_avg"], 0.1 * gr, rtol=1e-6)
    assert torch.allclose(out["exp_avg_sq"], 0.001 * gr * gr, rtol=1e-5)


def test_weight_decay_is_l2_not_decoupled():
    p = torch.full((4,), 2.0)
    out = adam_oracle.adam_step(p, torch.zeros(4), torch.zeros(4), torch.zeros(4), 1, 1e-2, weight_decay=0.5)
    # effective gradient 0.5 * 2 = 1 -> first step moves by lr
    assert torch.allclose(out["param"], torch.full((4,), 2.0 - 1e-2), rtol=1e-6)


def test_clip_coefficient_and_norm():
    assert adam_oracle.clip_coefficient(0.5, 1.0) == 1.0
    assert adam_oracle.clip_coefficient(4.0, 1.0) == pytest.approx(1.0 / (4.0 + 1e-6))
    gs = [torch.tensor([3.0, 4.0]), None, torch.tensor([[12.0]])]
    assert adam_oracle.grad_norm_squared(gs) == pytest.approx(169.0)
    total = torch.nn.utils.get_total_norm([g for g in gs if g is not None]).item()
    assert math.isclose(total**2, adam_oracle.grad_norm_squared(gs), rel_tol=1e-6)
