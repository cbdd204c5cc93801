"""Plain-PyTorch CPU restatement of the Qwen2.5-VL vision tower forward.

TEST INFRASTRUCTURE ONLY (see ``oracle/__init__.py``).  The functions take a
flat ``params`` dict whose keys are the reference's state-dict names, so the
product module's ``state_dict()`` can be fed in unchanged; gradients are
obtained with ``torch.autograd`` on those tensors.

All ``file:line`` citations are relative to the reference checkout
(``python/models/qwen2_5_vl/modeling_qwen2_5_vl.py`` unless another file is
named).  ``[tf]`` = transformers ``models/qwen2/modeling_qwen2.py``.

What pins each function (independently of this file's own formulae):

===================  =========================================================
``rot_pos_ids``      closed form per token (block row/col, dy, dx) checked by
                     brute-force raster scan in tests/test_oracle_planners.py
``window_index``     naive 2-D scan over all grids <= 12x12 merged units and
                     multi-frame cases; hand answer (1,16,16) -> 4x64;
                     permutation / same-window invariants
``cu_seqlens``       hand answers for video (per-frame segments)
``rms_norm``         ``torch.nn.functional.rms_norm`` (library routine)
``rope_apply``       2x2 rotation closed form, norm preservation, inverse
``attention``        ``F.scaled_dot_product_attention`` per segment
``mlp`` / ``merger`` ``F.silu`` / ``F.gelu`` / ``F.linear`` library routines
``patch_embed``      ``F.conv3d`` with kernel == stride vs. the GEMM form
``attn_block``       vectors written by the reference's own module
``block``            (tests/golden/reference_vectors.npz, made by
``tower_forward``    tests/golden/make_reference_vectors.py from an import of
                     modeling_qwen2_5_vl.py): output and every parameter
                     gradient of a 3-layer tower on ragged / video grids,
                     one attention module and one block alone, and the
                     configuration-1 tower (default initialisation, seed 0);
                     tests/test_oracle_golden.py also shows that the vectors
                     reject rotary-on-V, a wrong segment list, an unpermuted
                     rotary table and a missing reverse permutation, and
                     checks the zero-angle / depth-0 special cases against
                     ``F.multi_head_attention_forward`` and the bare merger.
===================  =========================================================
"""

from __future__ import annotations

import math
from dataclasses import dataclass, field
from typing import Dict, List, Sequence, Tuple

import torch
import torch.nn.functional as F


@dataclass
class OracleConfig:
    """Field names follow configuration_qwen2_5_vl.py:36-71."""

    depth: int = 32
    hidden_size: int = 1280
    intermediate_size: int = 3420
    num_heads: int = 16
    in_channels: int = 3
    patch_size: int = 14
    spatial_merge_size: int = 2
    temporal_patch_size: int = 2
    window_size: int = 112
    out_hidden_size: int = 3584
    fullatt_block_indexes: List[int] = field(default_factory=lambda: [7, 15, 23, 31])
    rms_norm_eps: float = 1e-6

    @property
    def head_dim(self) -> int:
        return self.hidden_size // self.num_heads


# --------------------------------------------------------------------------- planners


def rot_pos_ids(grid_thw: Sequence[Sequence[int]], merge: int) -> torch.Tensor:
    """(h, w) position of every patch in 2x2-merge-block order, repeated per frame.

    Follows rot_pos_emb, lines 841-864: reshape (h/m, m, w/m, m) -> permute
    (0, 2, 1, 3); the temporal index plays no part (``.repeat(t, 1)``).
    """
    out = []
    for t, h, w in grid_thw:
        t, h, w = int(t), int(h), int(w)
        hh = torch.arange(h).view(h // merge, merge, 1, 1).expand(h // merge, merge, w // merge, merge)
        ww = torch.arange(w).view(1, 1, w // merge, merge).expand(h // merge, merge, w // merge, merge)
        hh = hh.permute(0, 2, 1, 3).reshape(-1)
        ww = ww.permute(0, 2, 1, 3).reshape(-1)
        out.append(torch.stack([hh, ww], dim=-1).repeat(t, 1))
    return torch.cat(out, dim=0)


def rotary_table(grid_thw, merge: int, inv_freq: torch.Tensor) -> torch.Tensor:
    """[S, head_dim/2] angle table; lines 242-245 and 865-868.

    The arithmetic dtype is that of ``inv_freq`` (the reference's buffer is cast
    by ``model.to(bfloat16)``, so bf16 runs build this table in bf16).
    """
    ids = rot_pos_ids(grid_thw, merge)
    max_grid = max(max(int(h), int(w)) for _, h, w in grid_thw)
    seq = torch.arange(max_grid, dtype=inv_freq.dtype)
    freqs = torch.outer(seq, inv_freq)
    return freqs[ids].flatten(1)


def default_inv_freq(head_dim: int, theta: float = 10000.0) -> torch.Tensor:
    """lines 237-240 with dim = head_dim // 2 (line 829)."""
    dim = head_dim // 2
    return 1.0 / (theta ** (torch.arange(0, dim, 2, dtype=torch.float) / dim))


def window_index(grid_thw, merge: int, window_size: int, patch_size: int) -> Tuple[torch.Tensor, List[int]]:
    """Window permutation of the merged units and cumulative window lengths (in patches).

    Follows get_window_index, lines 870-909, including the padding rule
    ``pad = win - grid % win`` (a full extra band of empty windows when the grid
    divides evenly) and returns the raw cumulative list *with* its repeated
    entries; ``dedup_cu`` applies line 932's ``unique_consecutive``.
    """
    win = window_size // merge // patch_size
    unit = merge * merge
    idx_parts: List[torch.Tensor] = []
    cu: List[int] = [0]
    base = 0
    for t, h, w in grid_thw:
        t, gh, gw = int(t), int(h) // merge, int(w) // merge
        ph = win - gh % win
        pw = win - gw % win
        nh, nw = (gh + ph) // win, (gw + pw) // win
        grid = torch.full((t, gh + ph, gw + pw), -100, dtype=torch.long)
        grid[:, :gh, :gw] = torch.arange(t * gh * gw).view(t, gh, gw)
        tiles = grid.view(t, nh, win, nw, win).permute(0, 1, 3, 2, 4).reshape(t, nh * nw, win * win)
        counts = (tiles != -100).sum(-1).reshape(-1)
        flat = tiles.reshape(-1)
        idx_parts.append(flat[flat != -100] + base)
        running = cu[-1]
        for c in counts.tolist():
            running += c * unit
            cu.append(running)
        base += t * gh * gw
    return torch.cat(idx_parts), cu


def dedup_cu(cu: Sequence[int]) -> torch.Tensor:
    """line 927-932: int32 tensor with consecutive duplicates removed."""
    out = [cu[0]]
    for v in cu[1:]:
        if v != out[-1]:
            out.append(v)
    return torch.tensor(out, dtype=torch.int32)


def cu_seqlens(grid_thw) -> torch.Tensor:
    """lines 944-952: one attention segment per frame."""
    lens = []
    for t, h, w in grid_thw:
        lens += [int(h) * int(w)] * int(t)
    return torch.tensor([0] + list(torch.tensor(lens).cumsum(0).tolist()), dtype=torch.int32)


# --------------------------------------------------------------------------- arithmetic


def rms_norm(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    """[tf] lines 247-252: fp32 normalisation, cast back, then scale."""
    xf = x.to(torch.float32)
    var = xf.pow(2).mean(-1, keepdim=True)
    return weight * (xf * torch.rsqrt(var + eps)).to(x.dtype)


def rope_apply(x: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor) -> torch.Tensor:
    """lines 265-283 for one of q / k: x [S, H, d]; cos, sin [S, d]; fp32 inside."""
    xf = x.float()
    c = cos.unsqueeze(-2).float()
    s = sin.unsqueeze(-2).float()
    half = x.shape[-1] // 2
    rot = torch.cat((-xf[..., half:], xf[..., :half]), dim=-1)
    return (xf * c + rot * s).to(x.dtype)


def attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, cu: torch.Tensor, chunk: int = 2048) -> torch.Tensor:
    """Varlen non-causal attention, eager arithmetic of lines 298-321 per segment (449-468).

    q, k, v: [S, H, d].  Softmax in fp32, probabilities cast to the input dtype
    before the PV product.  Long segments are processed in query chunks; the
    softmax of every row is still exact over the whole segment.
    """
    scale = q.shape[-1] ** -0.5
    outs = []
    bounds = cu.tolist()
    for a, b in zip(bounds[:-1], bounds[1:]):
        if b == a:
            continue
        qs, ks, vs = (t[a:b].transpose(0, 1) for t in (q, k, v))  # [H, L, d]
        seg = []
        for r in range(0, b - a, chunk):
            w = torch.matmul(qs[:, r : r + chunk], ks.transpose(1, 2)) * scale
            w = F.softmax(w, dim=-1, dtype=torch.float32).to(q.dtype)
            seg.append(torch.matmul(w, vs))
        outs.append(torch.cat(seg, dim=1).transpose(0, 1))
    return torch.cat(outs, dim=0) if outs else q.new_empty(q.shape)


def mlp(x: torch.Tensor, p: Dict[str, torch.Tensor], prefix: str) -> torch.Tensor:
    """lines 203-204."""
    g = F.linear(x, p[prefix + "gate_proj.weight"], p[prefix + "gate_proj.bias"])
    u = F.linear(x, p[prefix + "up_proj.weight"], p[prefix + "up_proj.bias"])
    return F.linear(F.silu(g) * u, p[prefix + "down_proj.weight"], p[prefix + "down_proj.bias"])


def attn_block(x, p, prefix, cfg: OracleConfig, cu, cos, sin) -> torch.Tensor:
    """_forward_standard, lines 385-472."""
    S = x.shape[0]
    H, d = cfg.num_heads, cfg.head_dim
    q = F.linear(x, p[prefix + "q_proj.weight"], p[prefix + "q_proj.bias"]).view(S, H, d)
    k = F.linear(x, p[prefix + "k_proj.weight"], p[prefix + "k_proj.bias"]).view(S, H, d)
    v = F.linear(x, p[prefix + "v_proj.weight"], p[prefix + "v_proj.bias"]).view(S, H, d)
    q = rope_apply(q, cos, sin)
    k = rope_apply(k, cos, sin)
    o = attention(q, k, v, cu).reshape(S, H * d)
    return F.linear(o, p[prefix + "proj.weight"], p[prefix + "proj.bias"])


def block(x, p, i: int, cfg: OracleConfig, cu, cos, sin) -> torch.Tensor:
    """Qwen2_5_VLVisionBlock.forward, lines 776-792."""
    pre = f"blocks.{i}."
    x = x + attn_block(rms_norm(x, p[pre + "norm1.weight"], cfg.rms_norm_eps), p, pre + "attn.", cfg, cu, cos, sin)
    x = x + mlp(rms_norm(x, p[pre + "norm2.weight"], cfg.rms_norm_eps), p, pre + "mlp.")
    return x


def patch_embed(pixels: torch.Tensor, weight: torch.Tensor, cfg: OracleConfig) -> torch.Tensor:
    """lines 225-231 (Conv3d with kernel == stride, no bias)."""
    x = pixels.reshape(-1, cfg.in_channels, cfg.temporal_patch_size, cfg.patch_size, cfg.patch_size)
    stride = (cfg.temporal_patch_size, cfg.patch_size, cfg.patch_size)
    return F.conv3d(x.to(weight.dtype), weight, stride=stride).view(-1, cfg.hidden_size)


def merger(x: torch.Tensor, p: Dict[str, torch.Tensor], cfg: OracleConfig) -> torch.Tensor:
    """Qwen2_5_VLPatchMerger.forward, lines 248-262 (exact-erf GELU)."""
    unit = cfg.spatial_merge_size**2
    y = rms_norm(x, p["merger.ln_q.weight"], 1e-6).view(-1, cfg.hidden_size * unit)
    y = F.gelu(F.linear(y, p["merger.mlp.0.weight"], p["merger.mlp.0.bias"]))
    return F.linear(y, p["merger.mlp.2.weight"], p["merger.mlp.2.bias"])


def tower_forward(
    pixels: torch.Tensor,
    grid_thw: torch.Tensor,
    p: Dict[str, torch.Tensor],
    cfg: OracleConfig,
    inv_freq: torch.Tensor | None = None,
    return_hidden: bool = False,
):
    """Qwen2_5_VisionTransformerPretrainedModel.forward, lines 911-1070 (non-SP branch)."""
    grid = [[int(v) for v in row] for row in grid_thw.tolist()]
    unit = cfg.spatial_merge_size**2
    if inv_freq is None:
        inv_freq = default_inv_freq(cfg.head_dim)
    x = patch_embed(pixels, p["patch_embed.proj.weight"], cfg)
    S = x.shape[0]
    table = rotary_table(grid, cfg.spatial_merge_size, inv_freq)
    widx, cu_w_raw = window_index(grid, cfg.spatial_merge_size, cfg.window_size, cfg.patch_size)
    cu_w = dedup_cu(cu_w_raw)
    x = x.reshape(S // unit, unit, -1)[widx].reshape(S, -1)
    table = table.reshape(S // unit, unit, -1)[widx].reshape(S, -1)
    emb = torch.cat((table, table), dim=-1)
    cos, sin = emb.cos(), emb.sin()
    cu_full = cu_seqlens(grid)
    hiddens = []
    for i in range(cfg.depth):
        cu = cu_full if i in cfg.fullatt_block_indexes else cu_w
        x = block(x, p, i, cfg, cu, cos, sin)
        if return_hidden:
            hiddens.append(x)
    y = merger(x, p, cfg)
    y = y[torch.argsort(widx)]
    return (y, hiddens) if return_hidden else y


def max_rel_err(a: torch.Tensor, b: torch.Tensor) -> float:
    """max |a-b| / max |b| (the tolerance metric: 1e-4 in fp32, 2e-2 in bf16)."""
    a = a.detach().double().cpu()
    b = b.detach().double().cpu()
    denom = b.abs().max().item()
    if denom == 0.0:
        return (a - b).abs().max().item()
    return ((a - b).abs().max() / denom).item()


def rel_frobenius_err(a: torch.Tensor, b: torch.Tensor) -> float:
    """||a-b||_F / ||b||_F: a second metric beside max_rel_err, sensitive to errors spread over many small entries."""
    a = a.detach().double().cpu()
    b = b.detach().double().cpu()
    denom = b.norm().item()
    if denom == 0.0:
        return (a - b).norm().item()
    return ((a - b).norm() / denom).item()
