#!/usr/bin/env python3
"""Benchmark of the vision-tower hot path on one MI355X: forward + backward of the full-depth Qwen2.5-VL
vision tower (bf16).  Default workload: one 3584 x 3584 image = 65,536 patches with per-block activation
checkpointing (the largest single-GPU configuration); the 8-image ragged batch (cfg2) and the video (cfg5) are
timed beside it and reported under "other_workloads".

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload cfg3|cfg2|cfg5|cfg1|sample_yaml|one_896|one_224]

One "step" = zero_grad, forward, backward with a fixed upstream gradient (the optimizer is not part of the
path; "with_optimizer_step" reports the same loop with gradient norm, clipping and one Adam step added).  Inputs
and weights are resident in HBM before the timed region.  Prints ONE JSON line with the whole-job throughput
(patches/s), the roofline of the kernel that takes the most time in a step (per-launch durations from HIP events
on the compute stream), the attention MFMA utilisation (algorithmic FLOPs: the forward that a checkpointed block
re-runs in its backward adds time but no FLOPs), and the CPU baseline: the eager fp32 oracle timed on this box's
host cores on a bounded sample of the same workload.
"""

from __future__ import annotations

import argparse
import json
import os
import sys
import time
from pathlib import Path

ROOT = Path(__file__).resolve().parent
for _p in (ROOT, ROOT / "multimodal-training_amd"):
    if str(_p) not in sys.path:
        sys.path.insert(0, str(_p))

import numpy as np  # noqa: E402
import torch  # noqa: E402

PEAK_BF16_TFLOPS = 2500.0  # MI355X dense bf16 MFMA
PEAK_FP32_TFLOPS = 157.3
PEAK_HBM_GBS = 8000.0

FULL_TOWER = dict(depth=32, hidden_size=1280, intermediate_size=3420, num_heads=16, out_hidden_size=3584,
                  fullatt_block_indexes=[7, 15, 23, 31])


def make_workload(name: str):
    """Returns (description, config kwargs, dtype, grid_thw, seed, checkpointing)."""
    if name == "cfg2":
        g = torch.Generator(device="cpu").manual_seed(1)
        hw = 2 * torch.randint(16, 49, (8, 2), generator=g)  # sides of 28*k px, k in [16, 48], h and w independent
        grid = torch.cat([torch.ones(8, 1, dtype=torch.int64), hw], dim=1)
        return ("full Qwen2.5-VL vision tower (depth 32, 675M params), 8 ragged images, sides 448..1344 px (seed 1)",
                FULL_TOWER, torch.bfloat16, grid, 1, False)
    if name == "cfg3":
        return ("full tower, one 3584x3584 image = 65,536 patches, per-block activation checkpointing",
                FULL_TOWER, torch.bfloat16, torch.tensor([[1, 256, 256]]), 0, True)
    if name == "cfg5":
        return ("full tower, video 16 frames 448x784 = 8x32x56 = 14,336 patches (seed 3)",
                FULL_TOWER, torch.bfloat16, torch.tensor([[8, 32, 56]]), 3, False)
    if name == "sample_yaml":
        # the reference's own sample configuration (configs/sample.yaml:10,29,67-68): batch_size 4, min_pixels = max_pixels
        # = 802,816 (896 x 896 px = 64 x 64 patches per image), bfloat16, activation checkpointing on
        return ("full tower, 4 images 896x896 = 16,384 patches, per-block activation checkpointing (the reference's sample.yaml)",
                FULL_TOWER, torch.bfloat16, torch.tensor([[1, 64, 64]] * 4), 4, True)
    if name == "one_896":
        # the lower end of the batch sizes the reference's README names as usual (4-16 k tokens per step)
        return ("full tower, one 896x896 image = 4,096 patches, per-block activation checkpointing",
                FULL_TOWER, torch.bfloat16, torch.tensor([[1, 64, 64]]), 6, True)
    if name == "one_224":
        return ("full tower, one 224x224 image = 256 patches (a batch too small to fill the GPU: what a step costs at least)",
                FULL_TOWER, torch.bfloat16, torch.tensor([[1, 16, 16]]), 5, False)
    if name == "cfg1":
        kw = dict(FULL_TOWER, depth=4, out_hidden_size=2048, fullatt_block_indexes=[3])
        return ("reduced tower depth 4, fp32, 2 images 224x224", kw, torch.float32, torch.tensor([[1, 16, 16], [1, 16, 16]]), 0, False)
    raise SystemExit(f"unknown workload {name!r}")


def seg_sq_sum(cu: torch.Tensor) -> float:
    d = (cu[1:] - cu[:-1]).double()
    return float((d * d).sum())


def summarise_trace(records, cfg_kw, dtype):
    """Per-tag totals: launches, milliseconds, algorithmic FLOPs or bytes."""
    I = cfg_kw["intermediate_size"]
    ipad = (I + 7) // 8 * 8
    unpad = {ipad: I, 2 * ipad: 2 * I}
    out = {}
    for tag, info, e0, e1 in records:
        ms = e0.elapsed_time(e1)
        if tag.startswith("attn"):
            tag += "_window" if info["max_seqlen"] <= 64 else "_full"
        ent = out.setdefault(tag, {"launches": 0, "ms": 0.0, "ms_counted": 0.0, "flops": 0.0, "bytes": 0.0, "recomputed": 0})
        ent["launches"] += 1
        ent["ms"] += ms
        if info.get("recompute"):  # the forward a checkpointed block runs again: time, but no algorithmic work
            ent["recomputed"] += 1
            continue
        ent["ms_counted"] += ms
        if tag.startswith("gemm"):
            halves = 2.0 if tag.endswith("epi4") else 1.0  # SWIGLU: N counts one of the two weight matrices
            ent["flops"] += halves * 2.0 * info["M"] * unpad.get(info["N"], info["N"]) * unpad.get(info["K"], info["K"])
        elif tag.startswith("attn_fwd"):
            ent["flops"] += 4.0 * seg_sq_sum(info["cu"].cpu()) * info["head_dim"] * info["nheads"]
        elif tag.startswith("attn_bwd"):
            ent["flops"] += 10.0 * seg_sq_sum(info["cu"].cpu()) * info["head_dim"] * info["nheads"]
        elif tag == "rmsnorm_fwd":
            ent["bytes"] += 2.0 * info["rows"] * info["cols"] * info["esize"]
        elif tag == "rmsnorm_bwd":
            ent["bytes"] += (4.0 if info["add"] else 3.0) * info["rows"] * info["cols"] * info["esize"]
        elif tag == "rope":
            ent["bytes"] += 2.0 * info["rows"] * info["nheads"] * info["head_dim"] * info["esize"] + 2.0 * info["rows"] * info["head_dim"] * 4
        elif tag == "gather_rows":
            ent["bytes"] += 2.0 * info["rows"] * info["row_bytes"]
    return out


def measured_traffic_bytes(workload: str, tag: str):
    """HBM bytes per launch of a kernel group, as measured with rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE (two runs,
    each scaled by what the same counter reads for a 1 GiB device copy).  The figures live with the counter summaries
    they come from: a line ``traffic_bytes_per_launch <workload> <trace tag> <bytes>`` in a text file under profiles/.
    None when no summary holds such a line."""
    for f in sorted((ROOT / "profiles").glob("*.txt")):
        for line in f.read_text().splitlines():
            parts = line.split()
            if len(parts) >= 4 and parts[0] == "traffic_bytes_per_launch" and parts[1] == workload and parts[2] == tag:
                try:
                    return float(parts[3])
                except ValueError:
                    return None
    return None


KERNEL_NAMES = {
    "gemm_nn_epi0": "gemm_dl_kernel<TO, TA=false, TB=false, EPI=NONE>",
    "gemm_nn_epi1": "gemm_dl_kernel<TO, TA=false, TB=false, EPI=BIAS>",
    "gemm_nn_epi2": "gemm_dl_kernel<TO, TA=false, TB=false, EPI=BIAS_RES>",
    "gemm_nn_epi3": "gemm_dl_kernel<TO, TA=false, TB=false, EPI=BIAS_GELU>",
    "gemm_nn_epi4": "gemm_dl_kernel<TO, TA=false, TB=false, EPI=SWIGLU>",
    "gemm_nt_epi0": "gemm_dl_kernel<TO, TA=false, TB=true, EPI=NONE, MI16>",
    "gemm_nt_epi5": "gemm_dl_kernel<TO, TA=false, TB=true, EPI=SWIGLU_BWD>",
    "gemm_nt_epi6": "gemm_dl_kernel<TO, TA=false, TB=true, EPI=GELU_BWD>",
    "gemm_tt_epi0": "gemm_dl_kernel<TO, TA=true, TB=true, EPI=NONE, MI16> + splitk_reduce_kernel",
    "attn_fwd_full": "attn_fwd_x32<5> (segments >= 512 tokens), attn_fwd_mfma<5, 8, 32, true, 2, 4> (shorter)",
    "attn_bwd_full": "attn_delta_rows_kernel + attn_bwd_prepare_kernel + attn_bwd_dkdv_wide<5> + attn_bwd_dq_wide<5>",
    "attn_fwd_window": "attn_fwd_mfma<5, 2, 64, false, 2, 4>",
    "attn_bwd_window": "attn_bwd_window_mfma<5, 4, 2>",
}


def optimizer_leg(model, step, iters: int = 5):
    """The step after the path (not part of `value`): gradient norm, clipping and Adam over every parameter tensor.
    Multi-tensor kernels (one launch each) against what the reference calls on the same GPU: torch.optim.Adam(
    foreach=False) after a per-tensor gradient-scaling loop, and the per-tensor norm(2).item() loop."""
    from mi355_vit.optim import FusedAdam, grad_norm_squared

    params = [p for p in model.parameters() if p.requires_grad]
    n = sum(p.numel() for p in params)
    esize = params[0].element_size()
    step()  # fresh gradients
    torch.cuda.synchronize()

    def timed(fn, reps):
        fn()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(reps):
            fn()
        torch.cuda.synchronize()
        return 1000.0 * (time.perf_counter() - t0) / reps

    fused = FusedAdam(params, lr=1e-5)
    fused_ms = timed(lambda: fused.step(grad_scale=0.5), iters)
    norm_ms = timed(lambda: grad_norm_squared(params), iters)
    del fused
    ref = torch.optim.Adam(params, lr=1e-5, foreach=False)

    def ref_step():
        for p in params:
            p.grad.mul_(0.5)
        ref.step()

    ref_ms = timed(ref_step, 2)
    ref_norm_ms = timed(lambda: sum(p.grad.float().norm(2).item() ** 2 for p in params), 2)
    del ref
    traffic = n * esize * 8  # read p, g, m, v; write p, g (scaled), m, v
    return {"tensors": len(params), "parameters": n, "dtype": str(params[0].dtype).replace("torch.", ""),
            "adam_with_clip_ms": round(fused_ms, 3), "adam_with_clip_gbs": round(traffic / (fused_ms * 1e-3) / 1e9, 1),
            "grad_norm_ms": round(norm_ms, 3), "grad_norm_gbs": round(n * esize / (norm_ms * 1e-3) / 1e9, 1),
            "torch_adam_foreach_false_with_clip_ms": round(ref_ms, 3), "torch_norm_loop_ms": round(ref_norm_ms, 3)}


def handoff_leg(n_vision: int, hidden: int, dtype, iters: int = 20):
    """The step after the tower's output (not part of `value`): the [M, O] embeddings go into the <image> slots of a
    text sequence of M + 1024 tokens and the slot gradients come back.  Ranking + row-merge kernels against the
    reference's own calls on the same GPU (three counting guards with read-backs, masked_scatter, autograd)."""
    from mi355_vit.handoff import IMAGE_TOKEN_ID, extract_vision_grad, merge_vision_embeddings, prepare_vision_embeddings

    dev = torch.device("cuda:0")
    T = n_vision + 1024
    g = torch.Generator().manual_seed(0)
    ids = torch.randint(0, 1000, (1, T), generator=g)
    ids[0, 512 : 512 + n_vision] = IMAGE_TOKEN_ID
    labels = torch.randint(0, 1000, (1, T), generator=g)
    labels[ids == IMAGE_TOKEN_ID] = -100
    ids, labels = ids.to(dev), labels.to(dev)
    text = torch.randn(1, T, hidden, generator=g).to(dev, dtype).requires_grad_(True)
    vis = torch.randn(n_vision, hidden, generator=g).to(dev, dtype)
    gout = torch.randn(1, T, hidden, generator=g).to(dev, dtype)

    def ours():
        leaf = prepare_vision_embeddings(vis)
        merge_vision_embeddings(text, ids, leaf, labels).backward(gout)
        text.grad = None
        return extract_vision_grad(leaf)

    def reference_calls():
        leaf = prepare_vision_embeddings(vis)
        mask = (ids == IMAGE_TOKEN_ID).unsqueeze(-1).expand_as(text)
        n = (ids == IMAGE_TOKEN_ID).sum().item()
        assert n == leaf.shape[1] and bool(torch.all(labels[ids == IMAGE_TOKEN_ID] == -100))
        text.masked_scatter(mask, leaf.reshape(-1, hidden)).backward(gout)
        text.grad = None
        return extract_vision_grad(leaf)

    def timed(fn):
        fn()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(iters):
            fn()
        torch.cuda.synchronize()
        return 1000.0 * (time.perf_counter() - t0) / iters

    assert torch.equal(ours(), reference_calls())
    ours_ms, ref_ms = timed(ours), timed(reference_calls)
    esize = text.element_size()
    moved = (4 * T * hidden + 2 * n_vision * hidden) * esize  # merge fwd, zero-filling merge bwd, row gather bwd
    return {"tokens": T, "vision_rows": n_vision, "hidden": hidden, "fwd_bwd_ms": round(ours_ms, 3),
            "kernel_bytes_gbs": round(moved / (ours_ms * 1e-3) / 1e9, 1), "torch_masked_scatter_fwd_bwd_ms": round(ref_ms, 3)}


def input_leg(grid, dtype, iters: int = 20):
    """The step before the tower's input (not part of `value`): decoded uint8 frames of the workload's images ->
    pixel_values rows in the tower's dtype, one launch for the batch, against the same steps written with torch
    ops on the same GPU (rescale, normalise, reshape / permute per image, concatenate, cast)."""
    from mi355_vit.pixels import OPENAI_CLIP_MEAN, OPENAI_CLIP_STD, patchify

    dev = torch.device("cuda:0")
    g = torch.Generator().manual_seed(0)
    # a grid entry with t = 1 is a still image (one frame fills both halves of a row), t > 1 a video of 2 t frames
    frames = [torch.randint(0, 256, (1 if t == 1 else 2 * int(t), 14 * int(h), 14 * int(w), 3), generator=g, dtype=torch.uint8).to(dev)
              for t, h, w in grid.tolist()]
    rows = int(grid.prod(dim=1).sum())
    out = torch.empty((rows, 1176), dtype=dtype, device=dev)
    mean = torch.tensor(OPENAI_CLIP_MEAN, dtype=torch.float32, device=dev)
    std = torch.tensor(OPENAI_CLIP_STD, dtype=torch.float32, device=dev)

    def ours():
        return patchify(frames, dtype=dtype, out=out)[0]

    def torch_ops():
        parts = []
        for f in frames:
            n, h, w, _ = f.shape
            x = ((f.double() * (1.0 / 255.0)).float() - mean) / std
            x = x.permute(0, 3, 1, 2)
            if n % 2:
                x = torch.cat([x, x[-1:]], dim=0)
            x = x.reshape(x.shape[0] // 2, 2, 3, h // 28, 2, 14, w // 28, 2, 14).permute(0, 3, 6, 4, 7, 2, 1, 5, 8)
            parts.append(x.reshape(-1, 1176))
        return torch.cat(parts, dim=0).to(dtype)

    def timed(fn):
        fn()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(iters):
            fn()
        torch.cuda.synchronize()
        return 1000.0 * (time.perf_counter() - t0) / iters

    # the resize in front of it (PIL bicubic, bit-identical on the GPU): the workload's largest image from a decoded
    # frame 1.25 x its size, against Pillow on one host core (one call, bounded)
    from mi355_vit.pixels import resize_frames

    big = max(frames, key=lambda f: f.shape[1] * f.shape[2])
    th, tw = int(big.shape[1]), int(big.shape[2])
    raw = torch.randint(0, 256, (1, th * 5 // 4, tw * 5 // 4, 3), generator=g, dtype=torch.uint8)
    raw_dev = raw.to(dev)
    resize_ms = timed(lambda: resize_frames(raw_dev, th, tw))
    resize_gbs = (raw.numel() + th * tw * 3) / (resize_ms * 1e-3) / 1e9
    pil_ms = pil_same = None
    try:
        from PIL import Image
        t0 = time.perf_counter()
        ref = np.asarray(Image.fromarray(raw[0].numpy()).resize((tw, th), Image.Resampling.BICUBIC))
        pil_ms = 1000.0 * (time.perf_counter() - t0)
        pil_same = bool(np.array_equal(resize_frames(raw_dev, th, tw)[0].cpu().numpy(), ref))
    except ImportError:
        pass

    # the patch embedding straight from the frames (rows made inside the GEMM) against patchify + GEMM, bf16
    patch_embed = None
    if dtype == torch.bfloat16:
        from mi355_vit import ops
        from mi355_vit.pixels import pack_patch_embed_weight, patch_embed_frames

        w = (torch.randn(1280, 1176, generator=g) * 0.03).to(dev, torch.bfloat16)
        two_out = torch.empty((rows, 1280), dtype=dtype, device=dev)

        def fused():
            return patch_embed_frames(frames, pack_patch_embed_weight(w), dtype=dtype)[0]

        def two_kernels():
            ops.gemm(patchify(frames, dtype=dtype, out=out)[0], w, two_out)
            return two_out

        diff = float((fused().float() - two_kernels().float()).abs().max() / two_kernels().float().abs().max())
        fused_ms, two_ms = timed(fused), timed(two_kernels)
        patch_embed = {"embed_dim": 1280, "from_frames_ms": round(fused_ms, 3), "patchify_plus_gemm_ms": round(two_ms, 3),
                       "tflops_counted_on_k_1176": round(2.0 * rows * 1176 * 1280 / (fused_ms * 1e-3) / 1e12, 1),
                       "max_rel_diff": diff}

    same = bool(torch.equal(ours(), torch_ops()))  # bit for bit wherever torch's own kernels divide exactly
    max_diff = float((ours().float() - torch_ops().float()).abs().max())
    ours_ms, ref_ms = timed(ours), timed(torch_ops)
    frame_bytes = sum(f.numel() for f in frames)
    moved = frame_bytes + rows * 1176 * out.element_size()  # every input byte once, every output value once
    return {"images": len(frames), "rows": rows, "frame_bytes": frame_bytes, "out_dtype": str(dtype).replace("torch.", ""),
            "patchify_ms": round(ours_ms, 3), "algorithmic_gbs": round(moved / (ours_ms * 1e-3) / 1e9, 1),
            "torch_ops_ms": round(ref_ms, 3), "equals_torch_ops": same, "max_abs_diff_vs_torch_ops": max_diff,
            "resize": {"from": [int(raw.shape[1]), int(raw.shape[2])], "to": [th, tw], "filter": "bicubic", "gpu_ms": round(resize_ms, 3),
                       "algorithmic_gbs": round(resize_gbs, 1), "pillow_one_core_ms": None if pil_ms is None else round(pil_ms, 1),
                       "equals_pillow": pil_same},
            "patch_embed": patch_embed}


def cpu_baseline(cfg_kw, grid, seed, dtype, budget_s: float = 30.0):
    """Eager oracle (the reference's per-segment path, fp32) on the host cores, on a bounded sample of the workload.

    The sample is the two smallest images of the batch, or a 64 x 64-patch crop of the grid when a single image is
    larger than that (the eager path materialises [heads, L, L] scores: 256 GiB per full layer at L = 65,536).  Two
    towers are timed forward + backward: one windowed block, and one windowed + one full-attention block.  The time
    of the whole workload is extrapolated: everything but full attention grows linearly with the patch count, the
    full-attention excess with the sum of squared segment lengths."""
    from oracle import vit_oracle
    from oracle.vit_oracle import OracleConfig

    from mi355_vit.config import Qwen2_5_VLVisionConfig
    from mi355_vit.modeling import Qwen2_5_VisionTransformerPretrainedModel

    # every core this process may use: torch's default thread count follows OMP_NUM_THREADS (a GPU box gives a job its
    # share of the host that way) and is the machine's core count otherwise
    cores = torch.get_num_threads()
    order = sorted(range(grid.shape[0]), key=lambda i: int(grid[i].prod()))[:2]
    sub = grid[order].clone()
    sub[:, 0] = sub[:, 0].clamp(max=2)
    sub[:, 1:] = sub[:, 1:].clamp(max=64)
    S0 = int(sub.prod(dim=1).sum())
    S = int(grid.prod(dim=1).sum())

    def sq(gr):  # sum over attention segments (frames) of length^2
        return float((gr[:, 0] * (gr[:, 1] * gr[:, 2]) ** 2).sum())

    g = torch.Generator(device="cpu").manual_seed(seed)
    pixels = torch.randn(S0, 1176, generator=g)
    gout = torch.randn(S0 // 4, cfg_kw["out_hidden_size"], generator=g)

    def timed(depth, full):
        kw = dict(cfg_kw, depth=depth, fullatt_block_indexes=full)
        ocfg = OracleConfig(**{k: v for k, v in kw.items() if k in OracleConfig.__dataclass_fields__})
        torch.manual_seed(seed)
        ref = Qwen2_5_VisionTransformerPretrainedModel(Qwen2_5_VLVisionConfig(**kw))  # parameter container only (CPU)
        params = {k: v.detach().float().requires_grad_(True) for k, v in ref.state_dict().items()}
        best, t_start = None, time.perf_counter()
        for _ in range(2):
            for p in params.values():
                p.grad = None
            t0 = time.perf_counter()
            vit_oracle.tower_forward(pixels, sub, params, ocfg).backward(gout)
            dt_ = time.perf_counter() - t0
            best = dt_ if best is None else min(best, dt_)
            if time.perf_counter() - t_start > budget_s / 2:
                break
        return best

    n_full = len([i for i in cfg_kw["fullatt_block_indexes"] if i < cfg_kw["depth"]])
    if cfg_kw["depth"] < 2 or n_full == 0:
        t = timed(cfg_kw["depth"], list(cfg_kw["fullatt_block_indexes"]))
        return {"value": S0 / t, "unit": "patches/s", "cores": cores, "host_cores_visible": os.cpu_count(), "kind": "port",
                "sample": f"{S0} patches, whole tower fwd+bwd in fp32 took {t:.2f} s"}
    t_w = timed(1, [])      # patch embed + one windowed block + merger
    t_wf = timed(2, [1])    # ... + one full-attention block
    excess = max(t_wf - 2.0 * t_w, 0.0)  # what full attention costs beyond a windowed block at the sample's size
    n_win = cfg_kw["depth"] - n_full
    lin, quad = S / S0, sq(grid) / sq(sub)
    total = (n_win + n_full) * t_w * lin + n_full * excess * quad
    return {
        "value": S / total,
        "unit": "patches/s",
        "cores": cores,
        "host_cores_visible": os.cpu_count(),
        "kind": "port",
        "sample": f"grid {sub.tolist()} ({S0} patches) fwd+bwd in fp32: patch embed + 1 windowed block + merger {t_w:.2f} s, the same + 1 full block {t_wf:.2f} s; "
                  f"extrapolated to {cfg_kw['depth']} blocks ({n_full} full) of {S} patches: linear part x{lin:.2f}, full-attention excess "
                  f"x{quad:.1f} (sum of squared segment lengths) = {total:.0f} s per step",
    }


def main() -> None:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=10)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--workload", default="cfg3")
    ap.add_argument("--no-other-workloads", action="store_true", help="skip the cfg2 / cfg5 timings reported beside the metric")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-trace", action="store_true", help="skip the per-kernel event pass (for profiler runs)")
    ap.add_argument("--single-stream", action="store_true",
                    help="run weight / bias gradients in line on the main stream instead of on the second stream (for profiler "
                         "runs: kernels then never share the GPU, so their traced durations are their own)")
    ap.add_argument("--no-optimizer", action="store_true", help="skip the optimizer-step, hand-off and input-side measurements (reported beside the metric, never inside it)")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="run only a plain device copy of 1 GiB (8 launches) so that profiler byte counters can be scaled to a known size")
    args = ap.parse_args()
    if args.copy_calibration:
        src = torch.randn(1 << 28, device="cuda:0")  # 1 GiB of fp32
        dst = torch.empty_like(src)
        for _ in range(8):
            dst.copy_(src)
        torch.cuda.synchronize()
        print(json.dumps({"copy_calibration": {"launches": 8, "read_bytes_per_launch": src.numel() * 4, "written_bytes_per_launch": src.numel() * 4}}))
        return
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        raise SystemExit("bench.py measures the single-GPU hot path only: this build has no collectives; run with --gpus 1")
    if not torch.cuda.is_available():
        raise SystemExit("bench.py needs an MI355X (no CPU fallback)")

    from mi355_vit import ops
    from mi355_vit.config import Qwen2_5_VLVisionConfig
    from mi355_vit.modeling import Qwen2_5_VisionTransformerPretrainedModel

    if args.single_stream:
        ops.OVERLAP_WGRAD = False
    desc, cfg_kw, dtype, grid, seed, ckpt = make_workload(args.workload)
    dev = torch.device("cuda:0")
    torch.manual_seed(seed)
    model = Qwen2_5_VisionTransformerPretrainedModel(Qwen2_5_VLVisionConfig(**cfg_kw)).to(dtype).to(dev).train()
    if ckpt:
        model.gradient_checkpointing_enable()
    S = int((grid[:, 0] * grid[:, 1] * grid[:, 2]).sum())
    g = torch.Generator(device="cpu").manual_seed(seed)
    pixels = torch.randn(S, 1176, generator=g).to(dev)
    gout = torch.randn(S // 4, cfg_kw["out_hidden_size"], generator=g).to(dev, dtype)
    grid_dev = grid.to(dev)

    def step():
        model.zero_grad(set_to_none=True)
        # the grid goes in on the device and, as the trainer does, as the host copy it was made from (the model plans on
        # the host; without the copy it reads the device tensor back and the host waits for the GPU once per step)
        out = model(hidden_states=pixels, grid_thw=grid_dev, grid_thw_host=grid)
        out.backward(gout)

    def timed_steps(fn, warmup, steps, detail=None):
        """Wall-clock time of `steps` calls between two synchronisations.  With `detail` (a dict) also: a pair of HIP
        events on the compute stream around every call (the second stream joins the main one before a block hands
        its gradients back, so the closing event covers both) and the time the host needs to issue the calls."""
        for _ in range(warmup):
            fn()
        torch.cuda.synchronize()
        pairs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(steps)] if detail is not None else None
        t0 = time.perf_counter()
        for i in range(steps):
            if pairs:
                pairs[i][0].record()
            fn()
            if pairs:
                pairs[i][1].record()
        t_issued = time.perf_counter()
        torch.cuda.synchronize()
        t1 = time.perf_counter()
        if pairs:
            per = sorted(a.elapsed_time(b) for a, b in pairs)
            detail["event_ms_median"] = per[len(per) // 2] if len(per) % 2 else 0.5 * (per[len(per) // 2 - 1] + per[len(per) // 2])
            detail["event_ms_min"], detail["event_ms_max"] = per[0], per[-1]
            detail["host_issue_ms_per_step"] = 1000.0 * (t_issued - t0) / max(1, steps)
        return t1 - t0

    timing = {}
    elapsed = timed_steps(step, args.warmup, args.steps, timing)
    ms_per_step = 1000.0 * elapsed / max(1, args.steps)
    peak_mem_gb = torch.cuda.max_memory_allocated() / 2**30

    roofline, attn_util, breakdown = None, None, None
    if not args.no_trace:
        records: list = []
        ops.set_trace(records)
        step()
        torch.cuda.synchronize()
        ops.set_trace(None)
        summ = summarise_trace(records, cfg_kw, dtype)
        peak = PEAK_BF16_TFLOPS if dtype == torch.bfloat16 else PEAK_FP32_TFLOPS
        mfma_tags = {k: v for k, v in summ.items() if v["flops"] > 0}
        dom = max(mfma_tags, key=lambda k: mfma_tags[k]["ms"])
        d = mfma_tags[dom]
        ach = d["flops"] / (d["ms_counted"] * 1e-3) / 1e12  # per launch: recomputed launches are left out on both sides
        if dtype == torch.bfloat16:
            kernel_name = KERNEL_NAMES.get(dom, dom)
        else:  # the fp32 parity kernels: register-staged GEMM on v_mfma_f32_32x32x2_f32, one-lane-per-row attention
            kernel_name = f"gemm_kernel<float, float, ...> ({dom})" if dom.startswith("gemm") else f"attn_*_f32 ({dom})"
        roofline = {"bound": "mfma", "kernel": kernel_name, "launches_per_step": d["launches"],
                    "avg_launch_ms": d["ms"] / d["launches"], "achieved": ach, "peak": peak, "unit": "TFLOP/s",
                    "frac": ach / peak, "traffic": measured_traffic_bytes(args.workload, dom)}
        a_ms = sum(v["ms"] for t, v in summ.items() if t.startswith("attn"))
        a_fl = sum(v["flops"] for t, v in summ.items() if t.startswith("attn"))
        attn_util = a_fl / (a_ms * 1e-3) / 1e12 / peak if a_ms > 0 else None
        total_ms = sum(v["ms"] for v in summ.values())
        breakdown = {}
        for k, v in sorted(summ.items(), key=lambda kv: -kv[1]["ms"]):
            e = {"launches": v["launches"], "ms": round(v["ms"], 3), "share": round(v["ms"] / total_ms, 4)}
            if v["recomputed"]:
                e["recomputed_launches"] = v["recomputed"]
            if v["flops"]:  # per-launch rates: the launches of a re-run forward are left out on both sides
                e["tflops"] = round(v["flops"] / (v["ms_counted"] * 1e-3) / 1e12, 1)
            if v["bytes"]:
                e["gbs"] = round(v["bytes"] / (v["ms_counted"] * 1e-3) / 1e9, 1)
            breakdown[k] = e

    def side_leg(fn, *a):
        """The legs beside the metric never take the metric down with them: a failure is reported in their place."""
        try:
            return fn(*a)
        except Exception as e:  # noqa: BLE001
            return {"error": f"{type(e).__name__}: {e}"}

    def with_optimizer_leg():
        """The same loop with what follows the path in training: gradient norm, clipping coefficient and one Adam step
        over all parameters between two forward/backward passes (so every step runs on freshly updated weights)."""
        from mi355_vit.optim import FusedAdam, grad_norm_squared

        params = [p for p in model.parameters() if p.requires_grad]
        opt = FusedAdam(params, lr=1e-6)

        def train_step():
            step()
            norm = grad_norm_squared(params) ** 0.5
            opt.step(grad_scale=min(1.0, 1.0 / (norm + 1e-6)))

        n = max(2, min(args.steps, 5))
        t = timed_steps(train_step, 1, n)
        return {"steps": n, "ms_per_step": round(1000.0 * t / n, 3), "patches_per_s": round(S / (t / n), 1)}

    def other_workload(name, checkpointing=None):
        """Forward + backward of another configuration on the same tower (weights as they are), timing only.
        ``checkpointing`` overrides the configuration's own setting (None: as the configuration says)."""
        _, _, _, grid2, seed2, ckpt2 = make_workload(name)
        if checkpointing is not None:
            ckpt2 = checkpointing
        S2 = int(grid2.prod(dim=1).sum())
        g2 = torch.Generator(device="cpu").manual_seed(seed2)
        px = torch.randn(S2, 1176, generator=g2).to(dev)
        go = torch.randn(S2 // 4, cfg_kw["out_hidden_size"], generator=g2).to(dev, dtype)
        gd = grid2.to(dev)
        (model.gradient_checkpointing_enable if ckpt2 else model.gradient_checkpointing_disable)()

        def step2():
            model.zero_grad(set_to_none=True)
            model(hidden_states=px, grid_thw=gd, grid_thw_host=grid2).backward(go)

        torch.cuda.synchronize()
        torch.cuda.reset_peak_memory_stats()
        det = {}
        try:
            t = timed_steps(step2, 2, 5, det)
        finally:
            (model.gradient_checkpointing_enable if ckpt else model.gradient_checkpointing_disable)()
        return {"patches": S2, "grid_thw": grid2.tolist(), "activation_checkpointing": ckpt2, "steps": 5,
                "ms_per_step": round(1000.0 * t / 5, 3), "patches_per_s": round(S2 / (t / 5), 1),
                "event_ms_median": round(det["event_ms_median"], 3), "host_issue_ms_per_step": round(det["host_issue_ms_per_step"], 3),
                "peak_mem_gb": round(torch.cuda.max_memory_allocated() / 2**30, 2)}

    optimizer = handoff = input_side = with_opt = None
    others = None
    if not args.no_other_workloads and cfg_kw == FULL_TOWER:
        others = {name: side_leg(other_workload, name) for name in ("cfg2", "cfg3", "cfg5", "sample_yaml", "one_896") if name != args.workload}
        # the 65,536-patch image with every activation kept (no block is run twice): what 288 GB of HBM allow;
        # reported beside the metric, which stays on the configuration as it is named (checkpointing per block)
        others["cfg3_all_activations_kept"] = side_leg(other_workload, "cfg3", False)
    if not args.no_optimizer:
        with_opt = side_leg(with_optimizer_leg)
        optimizer = side_leg(optimizer_leg, model, step)
        handoff = side_leg(handoff_leg, S // 4, cfg_kw["out_hidden_size"], dtype)
        input_side = side_leg(input_leg, grid, dtype)

    cpu = None
    if not args.no_cpu_baseline:
        cpu = cpu_baseline(cfg_kw, grid, seed, dtype)

    result = {
        "metric": "vision fwd+bwd patches/sec on 1 MI355X; attention MFMA util % of bf16 peak",
        "value": S / (elapsed / max(1, args.steps)),
        "unit": "patches/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": ms_per_step,
        "timing": {"value_uses": "wall-clock mean of the timed steps between two synchronisations (ms_per_step)",
                   "event_ms_median": round(timing["event_ms_median"], 3), "event_ms_min": round(timing["event_ms_min"], 3),
                   "event_ms_max": round(timing["event_ms_max"], 3), "host_issue_ms_per_step": round(timing["host_issue_ms_per_step"], 3)},
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16" if dtype == torch.bfloat16 else "f32",
        "data": "synthetic",
        "config": {"workload": f"{args.workload}: {desc}", "patches": S, "grid_thw": grid.tolist(),
                   "activation_checkpointing": ckpt, "peak_mem_gb": round(peak_mem_gb, 2),
                   "streams": 2 if ops.OVERLAP_WGRAD else 1},
        "attention_mfma_util": attn_util,
        "roofline": roofline,
        "cpu_baseline": cpu,
        "other_workloads": others,
        "with_optimizer_step": with_opt,
        "optimizer_step": optimizer,
        "vision_text_handoff": handoff,
        "input_side": input_side,
        "kernel_breakdown": breakdown,
    }
    print(json.dumps(result))


if __name__ == "__main__":
    main()
