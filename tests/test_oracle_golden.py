"""The oracle (and the library's host planners) against vectors written by the reference's own Python.

tests/golden/reference_vectors.npz was produced by tests/golden/make_reference_vectors.py, which imports the
reference's modeling_qwen2_5_vl.py / sequence_parallel_utils.py in the build container and stores inputs and
outputs only.  These tests never import the reference.  They pin the composition functions of the oracle
(``attn_block``, ``block``, ``tower_forward``): each of the mutation tests below shows that a plausible mistake
(rotary embedding on V, the full-attention segment list on a windowed layer, a rotary table left in patch order,
a missing reverse permutation) is rejected by the stored vectors.
"""

from pathlib import Path

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle import sp_oracle, vit_oracle
from oracle.vit_oracle import OracleConfig

GOLDEN = Path(__file__).resolve().parent / "golden" / "reference_vectors.npz"
SMALL = dict(depth=3, hidden_size=32, intermediate_size=44, num_heads=2, out_hidden_size=16, fullatt_block_indexes=[1],
             patch_size=2, window_size=16)
CFG1 = dict(depth=4, hidden_size=1280, intermediate_size=3420, num_heads=16, out_hidden_size=2048, fullatt_block_indexes=[3])


@pytest.fixture(scope="module")
def vec():
    return np.load(GOLDEN, allow_pickle=False)


def rel(a: torch.Tensor, b: torch.Tensor) -> float:
    return vit_oracle.max_rel_err(a, b)


def frob(a: torch.Tensor, b: torch.Tensor) -> float:
    return vit_oracle.rel_frobenius_err(a, b)


def small_inputs(vec):
    params = {k[len("small/param/"):]: torch.from_numpy(vec[k]).clone().requires_grad_(True) for k in vec.files if k.startswith("small/param/")}
    grid = torch.from_numpy(vec["small/grid"])
    return params, grid, torch.from_numpy(vec["small/pixels"]), torch.from_numpy(vec["small/gout"])


def test_small_tower_output_and_every_gradient(vec):
    params, grid, pixels, gout = small_inputs(vec)
    cfg = OracleConfig(**SMALL)
    out = vit_oracle.tower_forward(pixels, grid, params, cfg, inv_freq=torch.from_numpy(vec["small/inv_freq"]))
    ref = torch.from_numpy(vec["small/out"])
    assert out.shape == ref.shape
    assert rel(out, ref) < 1e-5 and frob(out, ref) < 1e-5
    out.backward(gout)
    for name, p in params.items():
        g = torch.from_numpy(vec[f"small/grad/{name}"])
        assert rel(p.grad, g) < 2e-5 and frob(p.grad, g) < 2e-5, name


def _small_out(vec, **patches):
    params, grid, pixels, _ = small_inputs(vec)
    cfg = OracleConfig(**SMALL)
    with torch.no_grad():
        return vit_oracle.tower_forward(pixels, grid, params, cfg, inv_freq=torch.from_numpy(vec["small/inv_freq"]))


def test_the_vectors_reject_plausible_composition_mistakes(vec, monkeypatch):
    ref = torch.from_numpy(vec["small/out"])
    assert rel(_small_out(vec), ref) < 1e-5

    # (1) rotary embedding applied to V as well
    real_attention = vit_oracle.attention
    state = {}

    def rope_spy(x, cos, sin):
        state["cos"], state["sin"] = cos, sin
        return real_rope(x, cos, sin)

    real_rope = vit_oracle.rope_apply
    monkeypatch.setattr(vit_oracle, "rope_apply", rope_spy)
    monkeypatch.setattr(vit_oracle, "attention", lambda q, k, v, cu: real_attention(q, k, real_rope(v, state["cos"], state["sin"]), cu))
    assert rel(_small_out(vec), ref) > 1e-3
    monkeypatch.undo()

    # (2) the per-frame (full attention) segment list on every layer, and (3) the window list on every layer
    monkeypatch.setattr(vit_oracle, "dedup_cu", lambda cu: vit_oracle.cu_seqlens(vec["small/grid"].tolist()))
    assert rel(_small_out(vec), ref) > 1e-3
    monkeypatch.undo()
    real_dedup = vit_oracle.dedup_cu
    real_window_index = vit_oracle.window_index
    monkeypatch.setattr(vit_oracle, "cu_seqlens", lambda grid: real_dedup(real_window_index(grid, 2, 16, 2)[1]))
    assert rel(_small_out(vec), ref) > 1e-3
    monkeypatch.undo()

    # (4) rotary table left in patch order (not permuted with the tokens)
    real_table = vit_oracle.rotary_table

    def unpermuted_table(grid, merge, inv_freq):
        t = real_table(grid, merge, inv_freq)
        widx, _ = real_window_index(grid, merge, 16, 2)
        inv = torch.argsort(widx)
        return t.reshape(-1, merge * merge, t.shape[-1])[inv].reshape(t.shape)  # cancels the permutation applied later

    monkeypatch.setattr(vit_oracle, "rotary_table", unpermuted_table)
    assert rel(_small_out(vec), ref) > 1e-3
    monkeypatch.undo()

    # (5) the final reverse permutation dropped
    monkeypatch.setattr(torch, "argsort", lambda t, *a, **k: torch.arange(t.numel()))
    assert rel(_small_out(vec), ref) > 1e-3
    monkeypatch.undo()
    assert rel(_small_out(vec), ref) < 1e-5


def test_attention_module_and_block_alone(vec):
    params, _, _, _ = small_inputs(vec)
    cfg = OracleConfig(**SMALL)
    x = torch.from_numpy(vec["small/unit/x"])
    ang = torch.from_numpy(vec["small/unit/angles"])
    emb = torch.cat((ang, ang), dim=-1)
    cu = torch.from_numpy(vec["small/unit/cu"])
    with torch.no_grad():
        a = vit_oracle.attn_block(x, params, "blocks.0.attn.", cfg, cu, emb.cos(), emb.sin())
        b = vit_oracle.block(x, params, 2, cfg, cu, emb.cos(), emb.sin())
    assert rel(a, torch.from_numpy(vec["small/unit/attn0"])) < 1e-5
    assert rel(b, torch.from_numpy(vec["small/unit/block2"])) < 1e-5
    # zero rotary angles and a single segment: the attention module is torch's multi-head attention
    S, C, H = x.shape[0], cfg.hidden_size, cfg.num_heads
    one = torch.tensor([0, S], dtype=torch.int32)
    zero = torch.zeros(S, cfg.head_dim)
    w = torch.cat([params[f"blocks.0.attn.{n}_proj.weight"] for n in "qkv"]).detach()
    bias = torch.cat([params[f"blocks.0.attn.{n}_proj.bias"] for n in "qkv"]).detach()
    with torch.no_grad():
        mine = vit_oracle.attn_block(x, params, "blocks.0.attn.", cfg, one, zero.cos(), zero.sin())
        lib, _ = F.multi_head_attention_forward(x[:, None], x[:, None], x[:, None], C, H, w, bias, None, None, False, 0.0,
                                                params["blocks.0.attn.proj.weight"].detach(), params["blocks.0.attn.proj.bias"].detach(), need_weights=False)
    assert rel(mine, lib[:, 0]) < 1e-5


def test_depth_zero_tower_is_merger_of_patch_embed_in_natural_order(vec):
    params, grid, pixels, _ = small_inputs(vec)
    cfg = OracleConfig(**{**SMALL, "depth": 0, "fullatt_block_indexes": []})
    with torch.no_grad():
        out = vit_oracle.tower_forward(pixels, grid, params, cfg)
        x = pixels @ params["patch_embed.proj.weight"].reshape(cfg.hidden_size, -1).t()
        ref = vit_oracle.merger(x, params, cfg)  # rows of one merge unit are adjacent in patch order: no permutation at all
    assert rel(out, ref) < 1e-6


def test_configuration1_default_initialisation_output_and_gradients(vec):
    """Weights come from the product's module tree built under the same seed: their checksums must equal the
    reference's (same construction order, same default initialisers), and the oracle run on them must reproduce
    the reference's output and gradients."""
    from mi355_vit.config import Qwen2_5_VLVisionConfig
    from mi355_vit.modeling import Qwen2_5_VisionTransformerPretrainedModel

    torch.manual_seed(0)
    model = Qwen2_5_VisionTransformerPretrainedModel(Qwen2_5_VLVisionConfig(**CFG1))
    names = [str(n) for n in vec["cfg1/param_names"]]
    mine = dict(model.named_parameters())
    assert list(mine) == names
    sums = np.array([mine[n].detach().double().sum().item() for n in names])
    sumsq = np.array([mine[n].detach().double().pow(2).sum().item() for n in names])
    np.testing.assert_allclose(sums, vec["cfg1/param_sum"], rtol=1e-12, atol=1e-12)
    np.testing.assert_allclose(sumsq, vec["cfg1/param_sumsq"], rtol=1e-12)

    params = {k: v.detach().clone().requires_grad_(True) for k, v in model.state_dict().items()}
    g = torch.Generator().manual_seed(0)
    grid = torch.tensor([[1, 16, 16], [1, 16, 16]])
    pixels = torch.randn(512, 1176, generator=g)
    gout = torch.randn(128, 2048, generator=g)
    out = vit_oracle.tower_forward(pixels, grid, params, OracleConfig(**CFG1))
    ref_cols = torch.from_numpy(vec["cfg1/out_cols16"])
    scale = float(vec["cfg1/out_absmax"])
    assert ((out[:, ::16] - ref_cols).abs().max() / scale).item() < 1e-5
    assert frob(out[:, ::16], ref_cols) < 1e-5
    out.backward(gout)
    gsq = np.array([params[n].grad.double().pow(2).sum().item() for n in names])
    np.testing.assert_allclose(gsq, vec["cfg1/grad_sumsq"], rtol=1e-4)
    for key in vec.files:
        if key.startswith("cfg1/grad/"):
            n = key[len("cfg1/grad/"):]
            assert rel(params[n].grad, torch.from_numpy(vec[key])) < 2e-5, n
        if key.startswith("cfg1/grad_rows4/"):
            n = key[len("cfg1/grad_rows4/"):]
            got = params[n].grad.reshape(params[n].shape[0], -1)[:4]
            assert rel(got, torch.from_numpy(vec[key])) < 5e-5, n


def test_planners_window_index_rotary_table_and_cuts(vec):
    from mi355_vit import ops

    for i in range(int(vec["plan/n"])):
        grid = vec[f"plan/{i}/grid"].tolist()
        widx, cu_raw = vit_oracle.window_index(grid, 2, 112, 14)
        assert widx.tolist() == vec[f"plan/{i}/window_index"].tolist()
        assert list(cu_raw) == vec[f"plan/{i}/cu_window_raw"].tolist()
        assert vit_oracle.dedup_cu(cu_raw).tolist() == vec[f"plan/{i}/cu_window"].tolist()
        lib_idx, lib_cu = ops.window_index(torch.tensor(grid), 2, 112, 14)  # the library's closed-form planner
        assert lib_idx.tolist() == vec[f"plan/{i}/window_index"].tolist()
        assert lib_cu.tolist() == vec[f"plan/{i}/cu_window"].tolist()
        inv = vit_oracle.default_inv_freq(80)
        if f"plan/{i}/rotary_f32" in vec.files:
            assert torch.equal(vit_oracle.rotary_table(grid, 2, inv), torch.from_numpy(vec[f"plan/{i}/rotary_f32"]))
            ids = ops.rot_pos_ids(torch.tensor(grid), 2)
            assert torch.equal(ids, vit_oracle.rot_pos_ids(grid, 2))
        if f"plan/{i}/rotary_bf16_as_f32" in vec.files:  # the buffer after model.to(bfloat16): table built in bf16
            tb = vit_oracle.rotary_table(grid, 2, inv.to(torch.bfloat16))
            assert tb.dtype == torch.bfloat16 and torch.equal(tb.float(), torch.from_numpy(vec[f"plan/{i}/rotary_bf16_as_f32"]))
    for i in range(int(vec["cuts/n"])):
        args = vec[f"cuts/{i}/args"].tolist()
        n, sp, wl = args[0], args[1], args[2:]
        pos, idx = sp_oracle.window_cuts(n, sp, wl)
        assert list(pos) == vec[f"cuts/{i}/positions"].tolist() and list(idx) == vec[f"cuts/{i}/indices"].tolist()
        lpos, lidx = ops.sp_window_cuts(n, sp, wl)
        assert lpos == vec[f"cuts/{i}/positions"].tolist() and lidx == vec[f"cuts/{i}/indices"].tolist()
        assert sp_oracle.token_cuts(n, sp) == vec[f"cuts/{i}/token"].tolist() == ops.sp_token_cuts(n, sp)
