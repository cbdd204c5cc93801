"""Writes tests/golden/reference_vectors.npz from the reference's own Python (build container only).

Run once, where the reference checkout exists:  ``python tests/golden/make_reference_vectors.py [reference_root]``.
The reference module is imported, never copied: the file it writes holds inputs and outputs only.  The tests
that read the file (tests/test_oracle_golden.py) never import the reference.

Reference entry points exercised (python/models/qwen2_5_vl/):
  modeling_qwen2_5_vl.py   Qwen2_5_VisionTransformerPretrainedModel.{forward :911-1070, rot_pos_emb :841-868,
                           get_window_index :870-909}, Qwen2_5_VLVisionBlock.forward :776-792,
                           Qwen2_5_VLVisionAttention._forward_standard :385-472 (eager backend :298-321)
  sequence_parallel_utils.py  _compute_token_cut_positions :105-114, _compute_window_cut_positions :117-164

Vectors
  small/*   a tower small enough to store whole (hidden 32, 2 heads, depth 3, full attention at layer 1, 2 x 2-pixel
            patches): weights,
            pixels, upstream gradient, output, every parameter gradient, one attention module and one block on
            their own (window and full segment lists).  Grids: a ragged image whose windows do not divide, a
            two-frame video whose windows divide exactly (the extra empty band of windows), a narrow image.
  cfg1/*    the reduced-depth configuration-1 tower (hidden 1280, 16 heads, depth 4, full attention at layer 3,
            two 16x16-patch images), weights by default initialisation under seed 0: checksums of every weight,
            a column sample of the output and a few parameter gradients.
  plan/*    window permutations, cumulative window lengths, position ids, rotary tables (fp32 and the bf16
            buffer case) and sequence-parallel cut positions for edge-case inputs.
"""

from __future__ import annotations

import sys
from pathlib import Path

import numpy as np
import torch

HERE = Path(__file__).resolve().parent
OUT = HERE / "reference_vectors.npz"

# patch 2 x 2 (x 2 frames x 3 channels = 24 values per row) with 16-pixel windows keeps the 4 x 4-unit window geometry of
# the real model (112 / 2 / 14) while the pixel rows and the patch-embedding weight stay small
SMALL = dict(depth=3, hidden_size=32, intermediate_size=44, num_heads=2, out_hidden_size=16, fullatt_block_indexes=[1],
             patch_size=2, window_size=16)
SMALL_GRIDS = [[1, 6, 10], [2, 8, 8], [1, 12, 4]]
CFG1 = dict(depth=4, hidden_size=1280, intermediate_size=3420, num_heads=16, out_hidden_size=2048, fullatt_block_indexes=[3])
CFG1_GRIDS = [[1, 16, 16], [1, 16, 16]]
PLAN_GRIDS = [
    [[1, 16, 16]], [[1, 18, 22]], [[1, 8, 8]], [[3, 8, 12]], [[1, 2, 2]], [[1, 34, 16], [2, 8, 12]],
    [[1, 6, 10], [2, 8, 8], [1, 12, 4]], [[2, 10, 26]],
]
CUT_CASES = [  # (sample_len, sp, window lengths)
    (24, 2, [6, 4, 7, 7]), (10, 2, [6, 4]), (5, 4, [5]), (64, 4, [16, 16, 16, 16]), (100, 3, [64, 36]),
    (192, 8, [64, 64, 64]), (37, 5, [1, 2, 3, 4, 5, 6, 7, 9]), (256, 4, [64] * 4), (120, 4, [64, 32, 16, 8]),
]


def build_reference(ref_root: Path, kw: dict, seed: int):
    sys.path.insert(0, str(ref_root / "python"))
    from models.qwen2_5_vl.configuration_qwen2_5_vl import Qwen2_5_VLVisionConfig
    from models.qwen2_5_vl.modeling_qwen2_5_vl import Qwen2_5_VisionTransformerPretrainedModel

    cfg = Qwen2_5_VLVisionConfig(**kw)
    cfg._attn_implementation = "eager"
    torch.manual_seed(seed)
    model = Qwen2_5_VisionTransformerPretrainedModel(cfg)
    model.train()
    return model


def npf(t: torch.Tensor) -> np.ndarray:
    return t.detach().to(torch.float32).cpu().numpy().copy()


def main() -> None:
    ref_root = Path(sys.argv[1]) if len(sys.argv) > 1 else Path("/root/reference")
    out: dict = {}

    # ------------------------------------------------------------------ small tower, stored whole
    model = build_reference(ref_root, SMALL, seed=0)
    g = torch.Generator().manual_seed(1)
    for name, p in model.named_parameters():  # norm weights are all ones by default: perturb them so they matter
        if "norm" in name or "ln_q" in name:
            with torch.no_grad():
                p.add_(0.25 * torch.randn(p.shape, generator=g))
    grid = torch.tensor(SMALL_GRIDS, dtype=torch.int64)
    S = int((grid[:, 0] * grid[:, 1] * grid[:, 2]).sum())
    pixels = torch.randn(S, 3 * 2 * SMALL["patch_size"] ** 2, generator=g)
    gout = torch.randn(S // 4, SMALL["out_hidden_size"], generator=g)
    y = model(pixels, grid_thw=grid)
    y.backward(gout)
    out["small/grid"] = grid.numpy()
    out["small/pixels"] = npf(pixels)
    out["small/gout"] = npf(gout)
    out["small/out"] = npf(y)
    for name, p in model.named_parameters():
        out[f"small/param/{name}"] = npf(p)
        out[f"small/grad/{name}"] = npf(p.grad)
    out["small/inv_freq"] = npf(model.rotary_pos_emb.inv_freq)

    # one attention module and one block alone, on an explicit segment list and rotary angles
    Sx = 40
    x = torch.randn(Sx, SMALL["hidden_size"], generator=g)
    ang = torch.randn(Sx, SMALL["hidden_size"] // SMALL["num_heads"] // 2, generator=g)
    emb = torch.cat((ang, ang), dim=-1)
    cu = torch.tensor([0, 12, 13, 40], dtype=torch.int32)
    with torch.no_grad():
        a = model.blocks[0].attn(x, cu_seqlens=cu, position_embeddings=(emb.cos(), emb.sin()))
        b = model.blocks[2](x, cu_seqlens=cu, position_embeddings=(emb.cos(), emb.sin()))
    out["small/unit/x"], out["small/unit/angles"], out["small/unit/cu"] = npf(x), npf(ang), cu.numpy()
    out["small/unit/attn0"], out["small/unit/block2"] = npf(a), npf(b)

    # ------------------------------------------------------------------ configuration 1 (weights by seed)
    model = build_reference(ref_root, CFG1, seed=0)
    g = torch.Generator().manual_seed(0)
    grid = torch.tensor(CFG1_GRIDS, dtype=torch.int64)
    pixels = torch.randn(512, 1176, generator=g)
    gout = torch.randn(128, CFG1["out_hidden_size"], generator=g)
    y = model(pixels, grid_thw=grid)
    y.backward(gout)
    names = [n for n, _ in model.named_parameters()]
    out["cfg1/param_names"] = np.array(names)
    out["cfg1/param_sum"] = np.array([p.detach().double().sum().item() for _, p in model.named_parameters()])
    out["cfg1/param_sumsq"] = np.array([p.detach().double().pow(2).sum().item() for _, p in model.named_parameters()])
    out["cfg1/out_cols16"] = npf(y[:, ::16])
    out["cfg1/out_absmax"] = np.array(y.detach().abs().max().item())
    out["cfg1/grad_sumsq"] = np.array([p.grad.double().pow(2).sum().item() for _, p in model.named_parameters()])
    params = dict(model.named_parameters())
    for name in ("blocks.0.norm1.weight", "blocks.3.attn.q_proj.bias", "blocks.1.mlp.gate_proj.bias", "merger.mlp.2.bias", "merger.ln_q.weight"):
        out[f"cfg1/grad/{name}"] = npf(params[name].grad)
    for name in ("patch_embed.proj.weight", "blocks.2.mlp.down_proj.weight", "blocks.3.attn.k_proj.weight"):
        out[f"cfg1/grad_rows4/{name}"] = npf(params[name].grad.reshape(params[name].shape[0], -1)[:4])

    # ------------------------------------------------------------------ planners
    for i, gl in enumerate(PLAN_GRIDS):
        grid = torch.tensor(gl, dtype=torch.int64)
        widx, cu_w = model.get_window_index(grid)
        out[f"plan/{i}/grid"] = grid.numpy()
        out[f"plan/{i}/window_index"] = widx.numpy().astype(np.int64)
        out[f"plan/{i}/cu_window_raw"] = np.array(cu_w, dtype=np.int64)
        out[f"plan/{i}/cu_window"] = torch.unique_consecutive(torch.tensor(cu_w, dtype=torch.int32)).numpy()
        if i in (1, 3, 6):
            out[f"plan/{i}/rotary_f32"] = npf(model.rot_pos_emb(grid))
    out["plan/n"] = np.array(len(PLAN_GRIDS))
    import copy

    mb = copy.deepcopy(model.rotary_pos_emb).to(torch.bfloat16)  # what model.to(bfloat16) does to the buffer
    holder = copy.copy(model)
    holder.__dict__["_modules"] = dict(model._modules)
    holder._modules["rotary_pos_emb"] = mb
    for i in (1, 3):
        tb = holder.rot_pos_emb(torch.tensor(PLAN_GRIDS[i], dtype=torch.int64))
        assert tb.dtype == torch.bfloat16
        out[f"plan/{i}/rotary_bf16_as_f32"] = npf(tb)

    from models.qwen2_5_vl.sequence_parallel_utils import _compute_token_cut_positions, _compute_window_cut_positions

    for i, (n, sp, wl) in enumerate(CUT_CASES):
        pos, idx = _compute_window_cut_positions(n, sp, list(wl))
        out[f"cuts/{i}/args"] = np.array([n, sp] + list(wl), dtype=np.int64)
        out[f"cuts/{i}/positions"] = np.array(pos, dtype=np.int64)
        out[f"cuts/{i}/indices"] = np.array(idx, dtype=np.int64)
        out[f"cuts/{i}/token"] = np.array(_compute_token_cut_positions(n, sp), dtype=np.int64)
    out["cuts/n"] = np.array(len(CUT_CASES))

    np.savez_compressed(OUT, **out)
    print(f"wrote {OUT} ({OUT.stat().st_size / 1024:.0f} KiB, {len(out)} arrays)")


if __name__ == "__main__":
    main()
