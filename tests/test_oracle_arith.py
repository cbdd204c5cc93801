"""CPU tests pinning the oracle's floating-point functions against library routines and closed forms."""

import math

import torch
import torch.nn.functional as F

from oracle import vit_oracle
from oracle.vit_oracle import OracleConfig


def test_rms_norm_is_the_library_routine():
    x, w = torch.randn(7, 64, dtype=torch.float64), torch.randn(64, dtype=torch.float64)
    assert torch.allclose(vit_oracle.rms_norm(x, w, 1e-6), F.rms_norm(x, (64,), w, 1e-6), atol=1e-6)
    xb = torch.randn(5, 32).to(torch.bfloat16)
    wb = torch.randn(32).to(torch.bfloat16)
    out = vit_oracle.rms_norm(xb, wb, 1e-6)
    manual = wb * (xb.float() * torch.rsqrt(xb.float().pow(2).mean(-1, keepdim=True) + 1e-6)).to(torch.bfloat16)
    assert out.dtype == torch.bfloat16 and torch.equal(out, manual)


def test_rope_is_a_pairwise_rotation():
    S, H, d = 9, 3, 8
    x = torch.randn(S, H, d, dtype=torch.float64)
    ang = torch.randn(S, d // 2, dtype=torch.float64)
    emb = torch.cat([ang, ang], -1)
    y = vit_oracle.rope_apply(x.float(), emb.cos().float(), emb.sin().float()).double()
    for j in range(d // 2):
        a, b = x[..., j], x[..., j + d // 2]
        c, s = ang[:, j].cos()[:, None], ang[:, j].sin()[:, None]
        assert torch.allclose(y[..., j], a * c - b * s, atol=1e-5) and torch.allclose(y[..., j + d // 2], b * c + a * s, atol=1e-5)
    assert torch.allclose(y.pow(2).sum(-1), x.pow(2).sum(-1), rtol=1e-5)
    back = vit_oracle.rope_apply(y.float(), emb.cos().float(), (-emb).sin().float()).double()  # inverse rotation
    assert torch.allclose(back, x, atol=1e-5)


def test_attention_matches_sdpa_per_segment_and_chunking_is_exact():
    S, H, d = 50, 2, 16
    q, k, v = (torch.randn(S, H, d) for _ in range(3))
    cu = torch.tensor([0, 20, 21, 50], dtype=torch.int32)
    out = vit_oracle.attention(q, k, v, cu)
    for a, b in ((0, 20), (20, 21), (21, 50)):
        ref = F.scaled_dot_product_attention(q[a:b].transpose(0, 1)[None], k[a:b].transpose(0, 1)[None], v[a:b].transpose(0, 1)[None])[0].transpose(0, 1)
        assert torch.allclose(out[a:b], ref, atol=1e-5)
    assert torch.allclose(vit_oracle.attention(q, k, v, cu, chunk=7), out, atol=1e-6)
    # brute force on one row: softmax(q k^T / sqrt(d)) v
    w = torch.softmax((q[30, 1] @ k[21:50, 1].t()) / math.sqrt(d), -1)
    assert torch.allclose(out[30, 1], w @ v[21:50, 1], atol=1e-5)


def test_patch_embed_conv_equals_gemm_and_mlp_merger_formulae():
    cfg = OracleConfig(depth=1, hidden_size=32, intermediate_size=20, num_heads=2, out_hidden_size=24, fullatt_block_indexes=[0])
    w = torch.randn(32, 3, 2, 14, 14)
    px = torch.randn(12, 1176)
    assert torch.allclose(vit_oracle.patch_embed(px, w, cfg), px @ w.view(32, -1).t(), atol=1e-3)
    p = {"m.gate_proj.weight": torch.randn(20, 32), "m.gate_proj.bias": torch.randn(20), "m.up_proj.weight": torch.randn(20, 32),
         "m.up_proj.bias": torch.randn(20), "m.down_proj.weight": torch.randn(32, 20), "m.down_proj.bias": torch.randn(32)}
    x = torch.randn(5, 32)
    g = x @ p["m.gate_proj.weight"].t() + p["m.gate_proj.bias"]
    u = x @ p["m.up_proj.weight"].t() + p["m.up_proj.bias"]
    want = (g / (1 + torch.exp(-g)) * u) @ p["m.down_proj.weight"].t() + p["m.down_proj.bias"]
    assert torch.allclose(vit_oracle.mlp(x, p, "m."), want, atol=1e-4)
    pm = {"merger.ln_q.weight": torch.ones(32), "merger.mlp.0.weight": torch.randn(128, 128) * 0.1, "merger.mlp.0.bias": torch.zeros(128),
          "merger.mlp.2.weight": torch.randn(24, 128) * 0.1, "merger.mlp.2.bias": torch.randn(24)}
    xm = torch.randn(8, 32)
    z = F.rms_norm(xm, (32,), eps=1e-6).view(2, 128) @ pm["merger.mlp.0.weight"].t()
    gelu = 0.5 * z * (1 + torch.erf(z / math.sqrt(2)))
    assert torch.allclose(vit_oracle.merger(xm, pm, cfg), gelu @ pm["merger.mlp.2.weight"].t() + pm["merger.mlp.2.bias"], atol=1e-5)


def test_tower_shape_of_the_reference_smoke_case_and_checkpoint_free_gradients():
    """[192, 256] for grids (1,16,16),(1,16,32), hidden 256, 8 heads, depth 2, window 28 (reference smoke test)."""
    from mi355_vit.config import Qwen2_5_VLVisionConfig
    from mi355_vit.modeling import Qwen2_5_VisionTransformerPretrainedModel

    kw = dict(hidden_size=256, num_heads=8, depth=2, out_hidden_size=256, window_size=28, fullatt_block_indexes=[1])
    torch.manual_seed(0)
    model = Qwen2_5_VisionTransformerPretrainedModel(Qwen2_5_VLVisionConfig(**kw))  # CPU: parameters only
    params = {k: v.detach().clone().requires_grad_(True) for k, v in model.state_dict().items()}
    grid = torch.tensor([[1, 16, 16], [1, 16, 32]])
    out = vit_oracle.tower_forward(torch.randn(768, 1176), grid, params, OracleConfig(**kw))
    assert out.shape == (192, 256)
    out.square().mean().backward()
    assert all(p.grad is not None and torch.isfinite(p.grad).all() for p in params.values())
    assert vit_oracle.max_rel_err(torch.tensor([1.0, 2.0]), torch.tensor([1.0, 4.0])) == 0.5
