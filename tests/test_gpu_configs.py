"""The benchmark configurations run at their own grids, depth and sequence lengths (through the C ABI).

cfg2  depth-32 tower, bf16.  (a) The two smallest images of the seed-1 ragged batch against the fp32 oracle: output
      and all 518 parameter gradients, printed per parameter kind next to the error of the oracle itself evaluated in
      bf16 (tests/golden/bf16_oracle_errors.json, written by tests/golden/make_bf16_oracle_errors.py): what a bf16 run
      of the reference's own arithmetic shows against fp32.  The bar per kind is
      max(2e-2, 1.5 x the bf16 oracle's error for that kind) and the branch each kind took is printed.  (b) The whole
      eight-image batch (25,524 patches) through properties that need no O(L^2) host pass: finite, checkpointed == plain
      bit for bit, and batch == images run one at a time (outputs bit-equal row for row, parameter gradients equal
      to the sum of the single-image gradients within bf16 rounding of the sums).
cfg5  the 8 x 32 x 56 video: at depth 4 whole against the oracle, at depth 32 on two frames against the oracle (same
      bar as cfg2), and at depth 32 whole through the properties of (b), with the frames run one at a time.
cfg3  the 65,536-patch image at full size through properties that do not need an O(L^2) host pass: finite results,
      bounded peak memory, checkpointed and plain gradients bit-identical (depth 2 and depth 32), and the forward at
      depth 2 against the oracle on sampled merge units (the oracle's full-attention layer is evaluated for the
      sampled queries only).
"""

import collections
import copy
import importlib.util
import json
import re
from pathlib import Path

import pytest
import torch
import torch.nn.functional as F

from oracle import vit_oracle
from oracle.vit_oracle import OracleConfig, max_rel_err, rel_frobenius_err

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
GOLDEN = Path(__file__).resolve().parent / "golden"


def _cases():
    spec = importlib.util.spec_from_file_location("make_bf16_oracle_errors", GOLDEN / "make_bf16_oracle_errors.py")
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


CASES = _cases()
FULL = CASES.FULL
_build = CASES.build_model


def _ocfg(kw):
    return OracleConfig(**{k: v for k, v in kw.items() if k in OracleConfig.__dataclass_fields__})


def _oracle(model_cpu, kw, pixels, grid, gout, dtype=torch.float32):
    return CASES.run_oracle(model_cpu, kw, pixels, grid, gout, dtype)


def _gpu(model, pixels, grid, gout, keep_on_device=False):
    model.to(DEV).train()
    model.zero_grad(set_to_none=True)
    out = model(hidden_states=pixels.to(DEV), grid_thw=grid.to(DEV))
    out.backward(gout.to(device=DEV, dtype=out.dtype))
    torch.cuda.synchronize()
    if keep_on_device:
        return out.detach(), {n: p.grad.detach().clone() for n, p in model.named_parameters()}
    return out.detach().float().cpu(), {n: p.grad.detach().float().cpu() for n, p in model.named_parameters()}


def _errors(out, grads, ref_out, ref_grads):
    eo = (max_rel_err(out, ref_out), rel_frobenius_err(out, ref_out))
    worst = max(((max_rel_err(grads[n], ref_grads[n]), rel_frobenius_err(grads[n], ref_grads[n]), n) for n in grads), key=lambda t: t[0])
    worst_f = max(rel_frobenius_err(grads[n], ref_grads[n]) for n in grads)
    return eo, worst, worst_f


def _kind(name):
    return re.sub(r"blocks\.\d+\.", "blocks.*.", name)


def _check_against_oracle_with_bf16_bar(tag, case):
    """Output <= 2e-2 in both metrics.  Gradients: per parameter kind (q / k / v / proj / gate / up / down weights and
    biases, norms, patch embedding, merger) the worst error over the 32 blocks against the same figure of the bf16
    oracle; bar = max(2e-2, 1.5 x bf16 oracle), both metrics."""
    fixture = json.loads((GOLDEN / "bf16_oracle_errors.json").read_text())[case["name"]]
    assert fixture["grid_thw"] == case["grid"].tolist()
    model = _build(case["kw"], case["seed"])
    torch.set_num_threads(16)
    ref_out, ref_grads = _oracle(copy.deepcopy(model), case["kw"], case["pixels"].float(), case["grid"], case["gout"].float())
    out, grads = _gpu(model, case["pixels"], case["grid"], case["gout"])
    assert torch.isfinite(out).all() and all(torch.isfinite(v).all() for v in grads.values())
    eo_max, eo_frob = max_rel_err(out, ref_out), rel_frobenius_err(out, ref_out)
    S = int(case["grid"].prod(dim=1).sum())
    print(f"[{tag}] {S} patches, depth {case['kw']['depth']}: output max-rel {eo_max:.3e} frobenius {eo_frob:.3e} "
          f"(bf16 oracle: {fixture['output'][0]:.3e} / {fixture['output'][1]:.3e}); bar 2e-2", flush=True)
    assert eo_max < 2e-2 and eo_frob < 2e-2
    mine = collections.defaultdict(lambda: [0.0, 0.0, "", ""])
    theirs = collections.defaultdict(lambda: [0.0, 0.0])
    for n in grads:
        k = _kind(n)
        m, f = max_rel_err(grads[n], ref_grads[n]), rel_frobenius_err(grads[n], ref_grads[n])
        if m > mine[k][0]:
            mine[k][0], mine[k][2] = m, n
        if f > mine[k][1]:
            mine[k][1], mine[k][3] = f, n
        theirs[k][0] = max(theirs[k][0], fixture["gradients"][n][0])
        theirs[k][1] = max(theirs[k][1], fixture["gradients"][n][1])
    failures = []
    print(f"[{tag}] parameter gradients per kind, worst over the blocks: kernels vs fp32 oracle | bf16 oracle vs fp32 oracle | bar (branch)", flush=True)
    for k in sorted(mine, key=lambda k: -mine[k][0]):
        bar_m, bar_f = max(2e-2, 1.5 * theirs[k][0]), max(2e-2, 1.5 * theirs[k][1])
        branch = "2e-2" if bar_m == 2e-2 and bar_f == 2e-2 else "1.5 x bf16 oracle"
        print(f"[{tag}]   {k:32s} max-rel {mine[k][0]:.3e} ({mine[k][2]}) frob {mine[k][1]:.3e} | {theirs[k][0]:.3e} {theirs[k][1]:.3e} | "
              f"{bar_m:.3e} {bar_f:.3e} ({branch})", flush=True)
        if not (mine[k][0] < bar_m and mine[k][1] < bar_f):
            failures.append(k)
    assert not failures, f"gradient kinds beyond their bar: {failures}"


def test_cfg2_depth32_two_smallest_images():
    print("[case] cfg2: depth 32, bf16, two smallest images of the seed-1 batch", flush=True)
    _check_against_oracle_with_bf16_bar("cfg2", CASES.cfg2_two_smallest())


def test_cfg5_depth32_two_frames():
    print("[case] cfg5: depth 32, bf16, two frames of the 32 x 56 video", flush=True)
    _check_against_oracle_with_bf16_bar("cfg5", CASES.cfg5_two_frames())


def _whole_batch_properties(tag, kw, seed, grid, parts, pixel_seed):
    """Properties of a whole benchmark batch that need no host pass over it: finite results, checkpointed == plain bit
    for bit, and the batch equal to its parts run one at a time: outputs bit for bit (every row goes through the same
    kernels either way: a GEMM row does not depend on its batch, a segment does not depend on its neighbours), the
    parameter gradients equal to the sum of the parts' gradients within the bf16 rounding of those sums."""
    S = int(grid.prod(dim=1).sum())
    g = torch.Generator(device="cpu").manual_seed(pixel_seed)
    pixels = torch.randn(S, 1176, generator=g).to(torch.bfloat16)
    gout = torch.randn(S // 4, kw["out_hidden_size"], generator=g).to(torch.bfloat16)
    model = _build(kw, seed)
    out, grads = _gpu(model, pixels, grid, gout, keep_on_device=True)
    assert out.shape == (S // 4, kw["out_hidden_size"]) and torch.isfinite(out).all()
    assert all(torch.isfinite(v).all() for v in grads.values())
    model.gradient_checkpointing_enable()
    out_ck, grads_ck = _gpu(model, pixels, grid, gout, keep_on_device=True)
    assert torch.equal(out, out_ck)
    for n in grads:
        assert torch.equal(grads[n], grads_ck[n]), n
    del out_ck, grads_ck
    model.gradient_checkpointing_disable()
    sums = {n: torch.zeros_like(v, dtype=torch.float32) for n, v in grads.items()}
    row = 0
    for part in parts:
        n_rows = int(part.prod(dim=1).sum())
        o_p, g_p = _gpu(model, pixels[row:row + n_rows], part, gout[row // 4:(row + n_rows) // 4], keep_on_device=True)
        assert torch.equal(o_p, out[row // 4:(row + n_rows) // 4]), f"{tag}: rows {row}..{row + n_rows} differ between the batch and the part alone"
        for n in sums:
            sums[n] += g_p[n].float()
        row += n_rows
    assert row == S
    worst = max((max_rel_err(grads[n].float().cpu(), sums[n].cpu()), n) for n in grads)
    print(f"[{tag}] {S} patches, depth {kw['depth']}, {len(parts)} parts: outputs bit-equal; worst |batch gradient - sum of part gradients| / max "
          f"{worst[0]:.3e} ({worst[1]}); bar 1e-2 (each part's gradient is rounded to bf16 before the sum)", flush=True)
    assert worst[0] < 1e-2


def test_cfg2_whole_batch_depth32_properties():
    print("[case] cfg2: depth 32, bf16, the whole seed-1 batch of eight images", flush=True)
    hw, _ = CASES.cfg2_batch_grid()
    grid = torch.cat([torch.ones(8, 1, dtype=torch.int64), hw], dim=1)
    _whole_batch_properties("cfg2 whole", FULL, 1, grid, [grid[i:i + 1] for i in range(8)], pixel_seed=11)


def test_cfg5_whole_video_depth32_properties():
    print("[case] cfg5: depth 32, bf16, the whole 8 x 32 x 56 video, frames also one at a time", flush=True)
    grid = torch.tensor([[8, 32, 56]])
    _whole_batch_properties("cfg5 whole", FULL, 3, grid, [torch.tensor([[1, 32, 56]]) for _ in range(8)], pixel_seed=13)


def test_cfg5_video_depth4():
    print("[case] cfg5: video 8 x 32 x 56, depth 4 (full attention per frame at layer 3), bf16", flush=True)
    kw = dict(FULL, depth=4, fullatt_block_indexes=[3])
    grid = torch.tensor([[8, 32, 56]])
    S = 8 * 32 * 56
    g = torch.Generator(device="cpu").manual_seed(3)
    pixels = torch.randn(S, 1176, generator=g).to(torch.bfloat16)
    gout = torch.randn(S // 4, kw["out_hidden_size"], generator=g).to(torch.bfloat16)
    model = _build(kw, 3)
    torch.set_num_threads(16)
    ref_out, ref_grads = _oracle(copy.deepcopy(model), kw, pixels.float(), grid, gout.float())
    out, grads = _gpu(model, pixels, grid, gout)
    (eo_max, eo_frob), (gw_max, gw_frob, gw_name), g_frob = _errors(out, grads, ref_out, ref_grads)
    print(f"[cfg5] output max-rel {eo_max:.3e} frobenius {eo_frob:.3e}; worst gradient max-rel {gw_max:.3e} ({gw_name}), frobenius {g_frob:.3e}", flush=True)
    assert out.shape == (S // 4, 3584)
    assert eo_max < 2e-2 and eo_frob < 2e-2 and gw_max < 2e-2 and g_frob < 2e-2


def test_cfg3_65536_patch_image_depth32_checkpointed_equals_plain():
    print("[case] cfg3: one 256 x 256-patch image, bf16, depth 32, checkpointed and plain", flush=True)
    grid = torch.tensor([[1, 256, 256]])
    S, M = 65536, 16384
    g = torch.Generator(device="cpu").manual_seed(0)
    pixels = torch.randn(S, 1176, generator=g).to(torch.bfloat16)
    gout = torch.randn(M, FULL["out_hidden_size"], generator=g).to(torch.bfloat16)
    model = _build(FULL, 0)
    model.gradient_checkpointing_enable()
    torch.cuda.empty_cache()
    torch.cuda.reset_peak_memory_stats()
    out_ck, grads_ck = _gpu(model, pixels, grid, gout, keep_on_device=True)
    peak_ck = torch.cuda.max_memory_allocated() / 2**30
    assert out_ck.shape == (M, 3584) and torch.isfinite(out_ck).all()
    assert all(torch.isfinite(v).all() for v in grads_ck.values())
    assert not any((v == 0).all() for v in grads_ck.values()), "a parameter received no gradient"
    model.gradient_checkpointing_disable()
    torch.cuda.reset_peak_memory_stats()
    out_plain, grads_plain = _gpu(model, pixels, grid, gout, keep_on_device=True)
    peak_plain = torch.cuda.max_memory_allocated() / 2**30
    print(f"[cfg3] depth 32: peak memory {peak_ck:.1f} GiB checkpointed, {peak_plain:.1f} GiB plain", flush=True)
    assert torch.equal(out_plain, out_ck)
    for n in grads_plain:
        assert torch.equal(grads_plain[n], grads_ck[n]), n
    assert peak_ck < 24.0 and peak_plain < 120.0


def test_cfg3_65536_patch_image_properties():
    print("[case] cfg3: one 256 x 256-patch image, bf16, depth 2 (windowed + full layer), checkpointed and plain", flush=True)
    kw = dict(FULL, depth=2, fullatt_block_indexes=[1])
    grid = torch.tensor([[1, 256, 256]])
    S, M = 65536, 16384
    g = torch.Generator(device="cpu").manual_seed(0)
    pixels = torch.randn(S, 1176, generator=g).to(torch.bfloat16)
    gout = torch.randn(M, kw["out_hidden_size"], generator=g).to(torch.bfloat16)
    model = _build(kw, 0)
    cpu_model = copy.deepcopy(model)
    torch.cuda.reset_peak_memory_stats()
    out_plain, grads_plain = _gpu(model, pixels, grid, gout)
    model.gradient_checkpointing_enable()
    out_ck, grads_ck = _gpu(model, pixels, grid, gout)
    peak_gb = torch.cuda.max_memory_allocated() / 2**30
    print(f"[cfg3] peak memory {peak_gb:.2f} GiB at depth 2", flush=True)
    assert out_plain.shape == (M, 3584) and torch.isfinite(out_plain).all()
    assert all(torch.isfinite(v).all() for v in grads_plain.values())
    assert torch.equal(out_plain, out_ck)
    for n in grads_plain:
        assert torch.equal(grads_plain[n], grads_ck[n]), n
    assert peak_gb < 24.0

    # forward against the oracle on sampled merge units: layer 0 (windows) for every token, layer 1 (one 65,536-token
    # segment) for the sampled queries only
    torch.set_num_threads(16)
    ocfg = _ocfg(kw)
    p = {k: v.detach().float() for k, v in cpu_model.state_dict().items()}
    with torch.no_grad():
        x = vit_oracle.patch_embed(pixels.float(), p["patch_embed.proj.weight"], ocfg)
        table = vit_oracle.rotary_table(grid.tolist(), 2, cpu_model.rotary_pos_emb.inv_freq.detach().clone())
        widx, cu_raw = vit_oracle.window_index(grid.tolist(), 2, 112, 14)
        x = x.reshape(M, 4, -1)[widx].reshape(S, -1)
        table = table.reshape(M, 4, -1)[widx].reshape(S, -1)
        emb = torch.cat((table, table), dim=-1).float()
        cos, sin = emb.cos(), emb.sin()
        x = vit_oracle.block(x, p, 0, ocfg, vit_oracle.dedup_cu(cu_raw), cos, sin)
        units = torch.randint(0, M, (96,), generator=g)  # positions in window order
        rows = (units[:, None] * 4 + torch.arange(4)[None]).reshape(-1)
        n1 = vit_oracle.rms_norm(x, p["blocks.1.norm1.weight"], 1e-6)
        H, d = 16, 80
        q = F.linear(n1[rows], p["blocks.1.attn.q_proj.weight"], p["blocks.1.attn.q_proj.bias"]).view(-1, H, d)
        k = F.linear(n1, p["blocks.1.attn.k_proj.weight"], p["blocks.1.attn.k_proj.bias"]).view(S, H, d)
        v = F.linear(n1, p["blocks.1.attn.v_proj.weight"], p["blocks.1.attn.v_proj.bias"]).view(S, H, d)
        q = vit_oracle.rope_apply(q, cos[rows], sin[rows])
        k = vit_oracle.rope_apply(k, cos, sin)
        w = torch.softmax(torch.einsum("qhd,khd->hqk", q, k) * d**-0.5, dim=-1)
        o = torch.einsum("hqk,khd->qhd", w, v).reshape(-1, H * d)
        x1 = x[rows] + F.linear(o, p["blocks.1.attn.proj.weight"], p["blocks.1.attn.proj.bias"])
        x2 = x1 + vit_oracle.mlp(vit_oracle.rms_norm(x1, p["blocks.1.norm2.weight"], 1e-6), p, "blocks.1.mlp.")
        ref = vit_oracle.merger(x2, p, ocfg)  # [96, 3584], rows = sampled units in window order
    got = out_plain[widx[units]]  # the tower returns original order: unit at window position u is row widx[u]
    print(f"[cfg3] forward on 96 sampled merge units: max-rel {max_rel_err(got, ref):.3e} frobenius {rel_frobenius_err(got, ref):.3e}", flush=True)
    assert max_rel_err(got, ref) < 2e-2 and rel_frobenius_err(got, ref) < 2e-2
