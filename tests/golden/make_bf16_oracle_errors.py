"""Writes tests/golden/bf16_oracle_errors.json: how far the oracle itself, evaluated in bf16, lies from the oracle
in fp32 on the depth-32 test cases of tests/test_gpu_configs.py.

    python tests/golden/make_bf16_oracle_errors.py          (build container, CPU only, several minutes)

The figures are the bar for the depth-32 parameter gradients: a bf16 run of the reference's own arithmetic
(python/models/qwen2_5_vl/modeling_qwen2_5_vl.py, restated in oracle/vit_oracle.py) is no closer to fp32 than this,
so the kernels are asked to be no worse.  They are committed so that the bar does not depend on the host that runs
the GPU tests.  Per parameter: max-relative error ``max|a-b| / max|b|`` and relative Frobenius error of the gradient;
for the output the same two numbers.  The case builders below are imported by the test, so both sides see the same
inputs and weights.
"""

from __future__ import annotations

import json
import sys
from pathlib import Path

import torch

ROOT = Path(__file__).resolve().parents[2]
for _p in (ROOT, ROOT / "multimodal-training_amd"):
    if str(_p) not in sys.path:
        sys.path.insert(0, str(_p))

OUT = Path(__file__).resolve().parent / "bf16_oracle_errors.json"
FULL = dict(depth=32, hidden_size=1280, intermediate_size=3420, num_heads=16, out_hidden_size=3584, fullatt_block_indexes=[7, 15, 23, 31])


def build_model(kw, seed, dtype=torch.bfloat16):
    from mi355_vit.config import Qwen2_5_VLVisionConfig
    from mi355_vit.modeling import Qwen2_5_VisionTransformerPretrainedModel

    torch.manual_seed(seed)
    return Qwen2_5_VisionTransformerPretrainedModel(Qwen2_5_VLVisionConfig(**kw)).to(dtype)


def cfg2_batch_grid():
    """The seed-1 ragged batch of eight images (h and w drawn independently) and the generator after the draw."""
    g = torch.Generator(device="cpu").manual_seed(1)
    hw = 2 * torch.randint(16, 49, (8, 2), generator=g)
    return hw, g


def cfg2_two_smallest():
    hw, g = cfg2_batch_grid()
    order = sorted(range(8), key=lambda i: int(hw[i].prod()))[:2]
    grid = torch.cat([torch.ones(2, 1, dtype=torch.int64), hw[order]], dim=1)
    S = int(grid.prod(dim=1).sum())
    pixels = torch.randn(S, 1176, generator=g).to(torch.bfloat16)
    gout = torch.randn(S // 4, FULL["out_hidden_size"], generator=g).to(torch.bfloat16)
    return dict(name="cfg2_two_smallest_depth32", kw=FULL, seed=1, grid=grid, pixels=pixels, gout=gout)


def cfg5_two_frames():
    grid = torch.tensor([[2, 32, 56]])
    S = 2 * 32 * 56
    g = torch.Generator(device="cpu").manual_seed(3)
    pixels = torch.randn(S, 1176, generator=g).to(torch.bfloat16)
    gout = torch.randn(S // 4, FULL["out_hidden_size"], generator=g).to(torch.bfloat16)
    return dict(name="cfg5_two_frames_depth32", kw=FULL, seed=3, grid=grid, pixels=pixels, gout=gout)


CASES = [cfg2_two_smallest, cfg5_two_frames]


def run_oracle(model_cpu, kw, pixels, grid, gout, dtype):
    from oracle import vit_oracle
    from oracle.vit_oracle import OracleConfig

    ocfg = OracleConfig(**{k: v for k, v in kw.items() if k in OracleConfig.__dataclass_fields__})
    params = {k: v.detach().to(dtype).clone().requires_grad_(True) for k, v in model_cpu.state_dict().items()}
    inv_freq = model_cpu.rotary_pos_emb.inv_freq.detach().clone()
    out = vit_oracle.tower_forward(pixels.to(dtype), grid, params, ocfg, inv_freq=inv_freq)
    out.backward(gout.to(dtype))
    return out.detach().float(), {k: p.grad.float() for k, p in params.items()}


def main() -> None:
    import time

    from oracle.vit_oracle import max_rel_err, rel_frobenius_err

    result = {"torch": torch.__version__}
    for make in CASES:
        case = make()
        model = build_model(case["kw"], case["seed"])
        t0 = time.time()
        ref_out, ref_grads = run_oracle(model, case["kw"], case["pixels"].float(), case["grid"], case["gout"].float(), torch.float32)
        print(f"{case['name']}: fp32 oracle {time.time() - t0:.0f} s", flush=True)
        t0 = time.time()
        b_out, b_grads = run_oracle(model, case["kw"], case["pixels"], case["grid"], case["gout"], torch.bfloat16)
        print(f"{case['name']}: bf16 oracle {time.time() - t0:.0f} s", flush=True)
        result[case["name"]] = {
            "grid_thw": case["grid"].tolist(),
            "output": [max_rel_err(b_out, ref_out), rel_frobenius_err(b_out, ref_out)],
            "gradients": {n: [max_rel_err(b_grads[n], ref_grads[n]), rel_frobenius_err(b_grads[n], ref_grads[n])] for n in ref_grads},
        }
        worst = max(result[case["name"]]["gradients"].items(), key=lambda kv: kv[1][0])
        print(f"{case['name']}: output {result[case['name']]['output']}, worst gradient {worst}", flush=True)
    OUT.write_text(json.dumps(result, indent=0))
    print(f"wrote {OUT} ({OUT.stat().st_size} bytes)")


if __name__ == "__main__":
    main()
