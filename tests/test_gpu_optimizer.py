"""Parity of the multi-tensor optimizer step and gradient norm (through the C ABI) against the CPU oracle.

fp32 and bf16 results of the Adam step are compared bit for bit: the oracle restates torch.optim.Adam's
single-tensor path with torch's own association and fused multiply-adds and is itself pinned bit for bit against
torch.optim.Adam on the CPU (tests/test_oracle_adam.py).  Against torch.optim.Adam run on the GPU the tolerance is
1e-5 relative to the largest entry in fp32 and one bf16 step (2^-7) in bf16: torch's device kernels associate
addcmul / addcdiv differently from its host kernels.  The gradient norm squared is compared with an fp64 sum: 1e-6.
"""

import pytest
import torch

from oracle import adam_oracle

pytestmark = pytest.mark.gpu
DEV = "cuda:0"

SHAPES = [(37, 19), (8192 * 3 + 5,), (1280,), (1,), (5, 7, 3), (8192,), (300, 257)]


def _announce(msg):
    print(f"[case] {msg}", flush=True)


def _case(dtype, seed, steps):
    g = torch.Generator().manual_seed(seed)
    params = [(torch.randn(s, generator=g) * 0.05).to(dtype) for s in SHAPES]
    grads = [[(torch.randn(s, generator=g) * 10.0 ** float(torch.randint(-4, 1, (1,), generator=g))).to(dtype) for s in SHAPES]
             for _ in range(steps)]
    return params, grads


def _fused_run(params, grads_per_step, lr, wds, scales, misalign=False):
    from mi355_vit.optim import FusedAdam

    ps = []
    for p in params:
        if misalign:  # parameters that start one element into a buffer: no 16-byte alignment, scalar path of the kernel
            buf = torch.zeros(p.numel() + 1, dtype=p.dtype, device=DEV)
            view = buf[1:].view(p.shape)
            view.copy_(p)
            ps.append(torch.nn.Parameter(view))
        else:
            ps.append(torch.nn.Parameter(p.to(DEV)))
    opt = FusedAdam([{"params": [p], "weight_decay": wd} for p, wd in zip(ps, wds)], lr=lr)
    last_grads = None
    for grads, sc in zip(grads_per_step, scales):
        for p, g in zip(ps, grads):
            p.grad = g.to(DEV)
        opt.step(grad_scale=sc)
        last_grads = [p.grad.detach().cpu() for p in ps]
    return {"param": [p.detach().cpu() for p in ps], "exp_avg": [opt.state[p]["exp_avg"].cpu() for p in ps],
            "exp_avg_sq": [opt.state[p]["exp_avg_sq"].cpu() for p in ps], "grad": last_grads, "opt": opt}


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("wd", [0.0, 0.01])
@pytest.mark.parametrize("misalign", [False, True])
def test_fused_adam_bit_exact_against_oracle(dtype, wd, misalign):
    _announce(f"fused adam vs oracle {dtype} wd={wd} misalign={misalign}")
    steps, lr = 4, 1e-3
    params, grads = _case(dtype, 0, steps)
    wds = [wd if i % 2 == 0 else 0.0 for i in range(len(params))]
    scales = [1.0, 0.37, 1.0, 0.5]
    got = _fused_run(params, grads, lr, wds, scales, misalign)
    ref = adam_oracle.adam_run(params, grads, lr, wds, scales)
    for key in ("param", "exp_avg", "exp_avg_sq"):
        for i, (a, b) in enumerate(zip(got[key], ref[key])):
            assert a.dtype == b.dtype == dtype
            assert torch.equal(a, b), (key, SHAPES[i], (a.float() - b.float()).abs().max().item())
    # the scaled gradient is stored back, as Trainer._clip_gradients leaves it (last step: scale 0.5)
    for g_dev, g0 in zip(got["grad"], grads[-1]):
        assert torch.equal(g_dev, (g0.float() * torch.tensor(0.5)).to(dtype))
    for p in got["opt"].state:
        assert got["opt"].state[p]["step"].item() == steps and not got["opt"].state[p]["step"].is_cuda


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 1e-5), (torch.bfloat16, 2.0**-7)])
def test_fused_adam_against_torch_adam_on_gpu(dtype, tol):
    """The optimizer the reference builds, run by torch on the same GPU, for 5 steps with weight decay."""
    _announce(f"fused adam vs torch adam {dtype}")
    steps, lr = 5, 3e-3
    params, grads = _case(dtype, 1, steps)
    wds = [0.05 if i % 2 == 0 else 0.0 for i in range(len(params))]
    got = _fused_run(params, grads, lr, wds, [1.0] * steps)
    ps = [torch.nn.Parameter(p.to(DEV)) for p in params]
    opt = torch.optim.Adam([{"params": [p], "weight_decay": wd} for p, wd in zip(ps, wds)], lr=lr, foreach=False)
    for gs in grads:
        for p, g in zip(ps, gs):
            p.grad = g.to(DEV)
        opt.step()
    for key, ref in (("param", [p.detach().cpu() for p in ps]), ("exp_avg", [opt.state[p]["exp_avg"].cpu() for p in ps]),
                     ("exp_avg_sq", [opt.state[p]["exp_avg_sq"].cpu() for p in ps])):
        for i, (a, b) in enumerate(zip(got[key], ref)):
            err = (a.float() - b.float()).abs().max().item() / max(b.float().abs().max().item(), 1e-30)
            assert err <= tol, (key, SHAPES[i], err)
    # same state layout: each optimizer loads the other's state_dict
    sd = got["opt"].state_dict()
    assert set(sd["state"][0].keys()) == set(opt.state_dict()["state"][0].keys()) == {"step", "exp_avg", "exp_avg_sq"}
    opt.load_state_dict(sd)
    got["opt"].load_state_dict(opt.state_dict())


def test_fused_adam_skips_parameters_without_gradient_and_rejects_host_tensors():
    from mi355_vit.optim import FusedAdam

    a = torch.nn.Parameter(torch.ones(10, device=DEV))
    b = torch.nn.Parameter(torch.ones(10, device=DEV))
    opt = FusedAdam([a, b], lr=0.1)
    a.grad = torch.ones(10, device=DEV)
    opt.step()
    assert torch.allclose(a, torch.full_like(a, 0.9)) and torch.equal(b, torch.ones_like(b))
    assert b not in opt.state or len(opt.state[b]) == 0
    opt.step()  # nothing faults when only one of two tensors takes part, twice in a row
    c = torch.nn.Parameter(torch.ones(3))
    c.grad = torch.ones(3)
    with pytest.raises(RuntimeError, match="no CPU path"):
        FusedAdam([c]).step()
    e = torch.nn.Parameter(torch.ones(0, device=DEV))
    e.grad = torch.ones(0, device=DEV)
    FusedAdam([e]).step()  # empty tensors are skipped
    opt_none = FusedAdam([torch.nn.Parameter(torch.ones(4, device=DEV))])
    opt_none.step()  # no gradients at all: no launch


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_grad_norm_squared(dtype):
    from mi355_vit.optim import grad_norm_squared

    _announce(f"grad norm squared {dtype}")
    g = torch.Generator().manual_seed(2)
    shapes = SHAPES + [(1280, 3420), (2_000_003,)]
    params = []
    for s in shapes:
        p = torch.nn.Parameter(torch.zeros(s, dtype=dtype, device=DEV))
        p.grad = (torch.randn(s, generator=g) * 0.3).to(dtype).to(DEV)
        params.append(p)
    params.append(torch.nn.Parameter(torch.zeros(7, dtype=dtype, device=DEV)))  # no gradient
    got = grad_norm_squared(params)
    ref = adam_oracle.grad_norm_squared([p.grad.cpu() if p.grad is not None else None for p in params])
    assert abs(got - ref) <= 1e-6 * ref
    loop = sum(p.grad.float().norm(2).item() ** 2 for p in params if p.grad is not None)  # the reference's loop
    assert abs(got - loop) <= 1e-5 * loop
    assert grad_norm_squared([params[-1]]) == 0.0


def test_trainer_uses_the_multi_tensor_step():
    """VisionTrainer on the GPU: FusedAdam is built, one optimizer_step with clipping equals the oracle's update of
    every parameter from the same gradients (bit for bit), and the returned coefficient is the reference's formula."""
    from mi355_vit.optim import FusedAdam
    from mi355_vit.trainer import VisionTrainer

    cfg = dict(seed=0, parallelism="none", dtype="bfloat16", autocast=False, learning_rate=1e-3, weight_decay=0.05,
               warmup_ratio=0.0, warmup_steps=0, lr_scheduler_type="constant", num_iterations=4, max_grad_norm=1.0,
               activation_checkpointing=False, model_name=None,
               vision_config=dict(depth=2, hidden_size=256, intermediate_size=300, num_heads=8, out_hidden_size=256,
                                  window_size=56, fullatt_block_indexes=[1]),
               synthetic_grids=[[1, 16, 16], [1, 16, 32]])
    tr = VisionTrainer(cfg, rank=0)
    tr.build_model()
    tr.initialize_trainer()
    assert isinstance(tr.optimizer, FusedAdam) and len(tr.optimizer.param_groups) == 2
    out = tr.forward_step(0)["vision_embeddings"]
    tr.backward_step(torch.randn_like(out))
    named = dict(tr.model.named_parameters())
    before = {n: p.detach().cpu().clone() for n, p in named.items()}
    grads = {n: p.grad.detach().cpu().clone() for n, p in named.items()}
    norm_sq = tr.compute_grad_norm_contribution()["norm_sq"]
    assert abs(norm_sq - adam_oracle.grad_norm_squared(list(grads.values()))) <= 1e-6 * norm_sq
    gn = norm_sq**0.5
    coeff = tr.optimizer_step(global_grad_norm=gn)
    assert coeff == adam_oracle.clip_coefficient(gn, 1.0) and coeff < 1.0
    decay = {id(p) for p in tr.optimizer.param_groups[0]["params"]}
    for n, p in named.items():
        wd = 0.05 if id(p) in decay else 0.0
        assert (wd != 0.0) == (not any(x in f"model.{n}".lower() for x in ("bias", "norm", "ln_")))
        ref = adam_oracle.adam_step(before[n], grads[n], torch.zeros_like(before[n]), torch.zeros_like(before[n]), 1, 1e-3,
                                    weight_decay=wd, grad_scale=coeff)
        assert torch.equal(p.detach().cpu(), ref["param"]), n
        assert torch.equal(p.grad.cpu(), ref["grad"]), n


@pytest.mark.parametrize("dtype,copy_dtype", [(torch.bfloat16, torch.bfloat16), (torch.float32, torch.float32), (torch.float32, torch.bfloat16)])
def test_fused_adam_keeps_operand_copies_in_step(dtype, copy_dtype):
    """Parameters with a declared operand copy (plain, row-padded, at an offset inside a fused buffer, odd sizes):
    after every step the copy holds exactly the updated parameter (rounded once when the copy is bf16), the
    padding columns stay untouched, and the parameters equal those of a run without copies bit for bit."""
    from mi355_vit.optim import FusedAdam, attach_shadow

    _announce(f"operand copies {dtype} -> {copy_dtype}")
    g = torch.Generator().manual_seed(11)
    shapes = [(64, 3420), (300, 257), (1280,), (5, 7), (8192 * 2 + 3,), (96, 40)]
    params = [(torch.randn(s, generator=g) * 0.05).to(dtype) for s in shapes]
    plain = [torch.nn.Parameter(p.to(DEV)) for p in params]
    shadowed = [torch.nn.Parameter(p.to(DEV)) for p in params]
    bufs, views = [], []
    for i, p in enumerate(shadowed):
        if p.dim() == 2:
            pad = (0, 4, 7, 0, 0, 8)[i]
            buf = torch.full((p.shape[0] + 3, p.shape[1] + pad), 77.0, dtype=copy_dtype, device=DEV)
            view = buf[2 : 2 + p.shape[0], : p.shape[1]]
        else:
            buf = torch.full((p.numel() + 5,), 77.0, dtype=copy_dtype, device=DEV)
            view = buf[(0, 0, 4, 0, 1, 0)[i] :][: p.numel()]
        view.copy_(p.detach())
        attach_shadow(p, view)
        bufs.append(buf)
        views.append(view)
    o1, o2 = FusedAdam(plain, lr=1e-2, weight_decay=0.01), FusedAdam(shadowed, lr=1e-2, weight_decay=0.01)
    for step in range(3):
        for a, b in zip(plain, shadowed):
            gr = (torch.randn(a.shape, generator=g) * 0.1).to(dtype).to(DEV)
            a.grad, b.grad = gr, gr.clone()
        o1.step(grad_scale=0.5)
        o2.step(grad_scale=0.5)
        torch.cuda.synchronize()
        for a, b, view, buf in zip(plain, shadowed, views, bufs):
            assert torch.equal(a.detach(), b.detach())
            assert torch.equal(view, b.detach().to(copy_dtype))
            mask = torch.ones_like(buf, dtype=torch.bool)
            if buf.dim() == 2:
                mask[2 : 2 + b.shape[0], : b.shape[1]] = False
            else:
                off = view.data_ptr() - buf.data_ptr()
                mask[off // buf.element_size() :][: b.numel()] = False
            assert bool((buf[mask] == 77.0).all()), "the step wrote outside the copy"
    with pytest.raises(ValueError):
        attach_shadow(shadowed[0], torch.zeros(3, 3, device=DEV, dtype=copy_dtype))
