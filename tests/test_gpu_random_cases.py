"""Seeded random cases through the C ABI against the CPU oracles: shapes, layouts and options nobody picked by hand.

Each test draws its cases from ``random.Random(seed)``, announces a case before running it and checks it to the same
bar as the hand-written parity tests (bit-exact for byte / index work, 1e-4 in fp32, 2e-2 in bf16 otherwise)."""

import copy
import random

import numpy as np
import pytest
import torch

from oracle import pixels_oracle, resize_oracle, vit_oracle
from oracle.vit_oracle import OracleConfig, max_rel_err

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
TOL = {torch.float32: 1e-4, torch.bfloat16: 2e-2}


def _announce(msg):
    print(f"[case] {msg}", flush=True)


def _randn(shape, dtype, gen, scale=1.0):
    return (torch.randn(*shape, generator=gen) * scale).to(dtype)


# ------------------------------------------------------------------------------------------ GEMM
def _padded(rows, cols, dtype, gen, vec, extra):
    """A [rows, cols] view with unit column stride of a wider buffer (row pitch a multiple of the vector width)."""
    pitch = (cols + vec - 1) // vec * vec + vec * extra
    return _randn((rows, pitch), dtype, gen)[:, :cols]


def _to_device_keeping_pitch(t):
    buf = torch.zeros(t.shape[0], t.stride(0), dtype=t.dtype, device=DEV)
    view = buf[:, : t.shape[1]]
    view.copy_(t)
    return view


@pytest.mark.parametrize("seed", [0, 1])
def test_gemm_random_shapes_layouts_and_epilogues(seed):
    """out = epilogue(op(A) op(B)^T) for random M, N, K (tile multiples, single rows, odd edges), the three operand
    layouts the library builds, padded row pitches on every operand and on the output, bias / bias + residual /
    accumulate epilogues and K slices (with the plain, bias and bias + residual epilogues), against float32 matmul on the CPU; columns of the output buffer beyond N keep
    their contents."""
    from mi355_vit import _lib as E
    from mi355_vit import ops

    rnd = random.Random(9000 + seed)
    for case in range(40):
        dtype = rnd.choice([torch.bfloat16, torch.bfloat16, torch.float32])
        vec = 8 if dtype == torch.bfloat16 else 4
        M = rnd.choice([rnd.randint(1, 40), rnd.randint(1, 900), 256 * rnd.randint(1, 3)])
        N = rnd.choice([rnd.randint(1, 40), rnd.randint(1, 700), 256 * rnd.randint(1, 2)])
        ta, tb = rnd.choice([(False, False), (False, True), (True, True)])
        K = rnd.randint(1, 1200) if ta else vec * rnd.randint(1, 150)  # transposed operands: any contraction length
        epi = rnd.choice([E.EPI_NONE, E.EPI_NONE, E.EPI_BIAS, E.EPI_ACCUM] + ([] if tb else [E.EPI_BIAS_RES]))
        split = rnd.choice([1, 1, 2, 3]) if epi in (E.EPI_NONE, E.EPI_BIAS, E.EPI_BIAS_RES) and K >= 64 else 1
        out_dtype = dtype if dtype == torch.float32 else rnd.choice([torch.bfloat16, torch.float32])
        ldc = N + rnd.choice([0, 0, 3, 8])
        g = torch.Generator().manual_seed(1000 * seed + case)
        a = _padded(K, M, dtype, g, vec, rnd.randint(0, 2)) if ta else _padded(M, K, dtype, g, vec, rnd.randint(0, 2))
        b = _padded(K, N, dtype, g, vec, rnd.randint(0, 2)) if tb else _padded(N, K, dtype, g, vec, rnd.randint(0, 2))
        _announce(f"gemm {dtype}->{out_dtype} M={M} N={N} K={K} trans=({ta},{tb}) epi={epi} split_k={split} "
                  f"pitches a={a.stride(0)} b={b.stride(0)} out={ldc}")
        ref = (a.t() if ta else a).float() @ (b if tb else b.t()).float()
        kw = {}
        if epi in (E.EPI_BIAS, E.EPI_BIAS_RES):
            bias = _randn((N,), dtype, g)
            kw["bias"] = bias.to(DEV)
            ref = ref + bias.float()
        if epi == E.EPI_BIAS_RES:
            res = _padded(M, N, dtype, g, vec, rnd.randint(0, 1))
            kw["residual"] = _to_device_keeping_pitch(res)
            ref = ref + res.float()
        buf = torch.full((M, ldc), 777.0, dtype=out_dtype, device=DEV)
        out = buf[:, :N]
        if epi == E.EPI_ACCUM:
            c0 = _randn((M, N), out_dtype, g)
            out.copy_(c0)
            ref = ref + c0.float()
        ops.gemm(_to_device_keeping_pitch(a), _to_device_keeping_pitch(b), out, trans_a=ta, trans_b=tb, epilogue=epi,
                 split_k=split, **kw)
        assert max_rel_err(out, ref) < (2e-5 if dtype == torch.float32 else TOL[torch.bfloat16] / 2)
        assert bool((buf[:, N:] == 777.0).all())


# ------------------------------------------------------------------------------------------ attention
@pytest.mark.parametrize("seed", [0, 1])
def test_attention_random_segment_layouts(seed):
    """Forward, log-sum-exp, dQ, dK, dV for random segment layouts (windows, mid-length, long and mixed batches; one to
    four heads; head_dim 32 / 64 / 80 / 128; q, k, v packed in one buffer or apart) against the oracle."""
    from mi355_vit import ops

    rnd = random.Random(7000 + seed)
    for case in range(25):
        d = rnd.choice([80, 80, 80, 64, 32, 128])
        H = rnd.randint(1, 4)
        kind = rnd.choice(["windows", "mid", "long", "mixed"])
        if kind == "windows":
            seg = [rnd.randint(1, 64) for _ in range(rnd.randint(1, 12))]
        elif kind == "mid":
            seg = [rnd.randint(1, 520) for _ in range(rnd.randint(1, 5))]
        elif kind == "long":
            seg = [rnd.randint(500, 1500) for _ in range(rnd.randint(1, 3))]
        else:
            seg = [rnd.choice([rnd.randint(1, 64), rnd.randint(65, 600), rnd.randint(512, 1300)]) for _ in range(rnd.randint(2, 5))]
        dtype = rnd.choice([torch.float32, torch.bfloat16])
        packed = rnd.random() < 0.5
        _announce(f"attention {dtype} segments={seg} H={H} d={d} packed={packed}")
        S, C = sum(seg), H * d
        g = torch.Generator().manual_seed(1000 * seed + case)
        cu = torch.tensor([0] + list(np.cumsum(seg)), dtype=torch.int32)
        if packed:
            qkv = _randn((S, 3 * C), dtype, g)
            q, k, v = qkv[:, :C], qkv[:, C : 2 * C], qkv[:, 2 * C :]
            qkv_g = qkv.to(DEV)
            qg, kg, vg = qkv_g[:, :C], qkv_g[:, C : 2 * C], qkv_g[:, 2 * C :]
        else:
            q, k, v = (_randn((S, C), dtype, g) for _ in range(3))
            qg, kg, vg = q.to(DEV), k.to(DEV), v.to(DEV)
        do = _randn((S, C), dtype, g)
        o, lse = ops.attn_fwd(qg, kg, vg, cu.to(DEV), max(seg), H, d, d**-0.5)
        qr, kr, vr = (t.float().reshape(S, H, d).clone().requires_grad_(True) for t in (q, k, v))
        o_ref = vit_oracle.attention(qr, kr, vr, cu)
        assert max_rel_err(o, o_ref.reshape(S, C)) < TOL[dtype]
        lse_ref = torch.cat([torch.logsumexp(torch.einsum("qhd,khd->hqk", qr[a:b], kr[a:b]) * d**-0.5, dim=-1)
                             for a, b in zip(cu[:-1].tolist(), cu[1:].tolist())], dim=1).detach()
        # bf16 kernels round the pre-scaled queries (q * scale * log2 e) to bf16 once more: a score, and with it the
        # log-sum-exp of a short segment, moves by a few 1e-3
        at = 8e-3 if dtype == torch.bfloat16 else 1e-5
        assert torch.allclose(lse.cpu(), lse_ref, rtol=at, atol=at)
        o_ref.backward(do.float().reshape(S, H, d))
        dq, dk, dv = (torch.full((S, C), float("nan"), dtype=dtype, device=DEV) for _ in range(3))
        ops.attn_bwd(qg, kg, vg, o, do.to(DEV), lse, cu.to(DEV), max(seg), H, d, d**-0.5, dq, dk, dv)
        for name, got, ref in (("dq", dq, qr.grad), ("dk", dk, kr.grad), ("dv", dv, vr.grad)):
            assert max_rel_err(got, ref.reshape(S, C)) < TOL[dtype], name


# ------------------------------------------------------------------------------------------ tower
def test_tower_random_configurations():
    """Whole towers of random geometry (head_dim 32 / 64 / 80, 2-16 heads, odd intermediate sizes, depth 1-3 with or
    without a full-attention layer, 1-4 images and videos of random even grids, float32 or bfloat16, with or without
    per-block checkpointing): output and every parameter gradient against the float32 oracle on the same weights."""
    from mi355_vit.config import Qwen2_5_VLVisionConfig
    from mi355_vit.modeling import Qwen2_5_VisionTransformerPretrainedModel

    rnd = random.Random(1000)
    for case in range(16):
        hd = rnd.choice([80, 80, 64, 32])
        heads = rnd.choice([2, 4, 16]) if hd == 80 else rnd.choice([2, 4, 8])
        hidden = hd * heads
        inter = rnd.choice([2 * hidden + 4, 300, 3420 if hidden == 1280 else hidden + 12])
        out_hidden = rnd.choice([64, 128, 520])
        depth = rnd.randint(1, 3)
        full = sorted(rnd.sample(range(depth), rnd.randint(0, 1)))
        kw = dict(depth=depth, hidden_size=hidden, intermediate_size=inter, num_heads=heads, out_hidden_size=out_hidden,
                  fullatt_block_indexes=full)
        grid = torch.tensor([[rnd.choice([1, 1, 1, 2, 3]), 2 * rnd.randint(1, 18), 2 * rnd.randint(1, 18)]
                             for _ in range(rnd.randint(1, 4))])
        if int(grid.prod(dim=1).sum()) > 3000:
            grid = grid[:1]
        S = int(grid.prod(dim=1).sum())
        dtype = rnd.choice([torch.float32, torch.bfloat16])
        checkpoint = rnd.random() < 0.5
        _announce(f"tower {kw} grid={grid.tolist()} {dtype} checkpoint={checkpoint}")
        torch.manual_seed(case)
        model = Qwen2_5_VisionTransformerPretrainedModel(Qwen2_5_VLVisionConfig(**kw)).to(dtype)
        if checkpoint:
            model.gradient_checkpointing_enable()
        g = torch.Generator().manual_seed(case)
        pixels = _randn((S, 1176), dtype, g)
        gout = _randn((S // 4, out_hidden), dtype, g)
        cpu = copy.deepcopy(model)
        params = {k: v.detach().float().clone().requires_grad_(True) for k, v in cpu.state_dict().items()}
        ocfg = OracleConfig(**{k: v for k, v in kw.items() if k in OracleConfig.__dataclass_fields__})
        ref = vit_oracle.tower_forward(pixels.float(), grid, params, ocfg, inv_freq=cpu.rotary_pos_emb.inv_freq.detach().clone())
        ref.backward(gout.float())
        model.to(DEV).train()
        out = model(hidden_states=pixels.to(DEV), grid_thw=grid.to(DEV))
        out.backward(gout.to(DEV))
        assert max_rel_err(out, ref.detach()) < TOL[dtype]
        worst = max((max_rel_err(p.grad, params[n].grad), n) for n, p in model.named_parameters())
        assert worst[0] < TOL[dtype], worst


# ------------------------------------------------------------------------------------------ input side
def test_input_side_random_frames_and_resizes():
    """Random batches of images and videos through patchify (bit-exact against the oracle) and the fused patch
    embedding (against the oracle's rows times the weight), and random resizes (both filters, up and down, 1 or 3
    frames, sizes down to one pixel) bit-exact against the oracle's restatement of Pillow."""
    from mi355_vit import pixels

    rnd = random.Random(5000)
    for case in range(16):
        rng = np.random.default_rng(5000 + case)
        shapes = [(rnd.choice([1, 1, 2, 3, 4]), 28 * rnd.randint(1, 8), 28 * rnd.randint(1, 8)) for _ in range(rnd.randint(1, 5))]
        _announce(f"frames {shapes}")
        images = [rng.integers(0, 256, size=(f, h, w, 3), dtype=np.uint8) for f, h, w in shapes]
        frames = [torch.from_numpy(im).to(DEV) for im in images]
        got, grid = pixels.patchify(frames)
        ref, ref_grid = pixels_oracle.patchify_batch(images)
        assert grid.tolist() == ref_grid.tolist()
        assert np.array_equal(got.cpu().numpy().view(np.uint32), ref.view(np.uint32))
        embed = rnd.choice([64, 200, 1280])
        w = _randn((embed, 1176), torch.bfloat16, torch.Generator().manual_seed(case), 0.03).to(DEV)
        fused, _ = pixels.patch_embed_frames(frames, pixels.pack_patch_embed_weight(w))
        want = torch.from_numpy(ref).to(torch.bfloat16).float() @ w.float().cpu().t()
        assert max_rel_err(fused, want) < TOL[torch.bfloat16] / 2

        ih, iw = rnd.randint(5, 400), rnd.randint(5, 400)
        oh = rnd.choice([rnd.randint(1, 300), 28 * rnd.randint(1, 10)])
        ow = rnd.choice([rnd.randint(1, 300), 28 * rnd.randint(1, 10)])
        filt, nf = rnd.choice(["bicubic", "bilinear"]), rnd.choice([1, 1, 3])
        _announce(f"resize {nf} x {ih} x {iw} -> {oh} x {ow} {filt}")
        img = rng.integers(0, 256, size=(nf, ih, iw, 3), dtype=np.uint8)
        resized = pixels.resize_frames(torch.from_numpy(img).to(DEV), oh, ow, filt).cpu().numpy()
        assert np.array_equal(resized, np.stack([resize_oracle.pil_resize(img[i], oh, ow, filt) for i in range(nf)]))
