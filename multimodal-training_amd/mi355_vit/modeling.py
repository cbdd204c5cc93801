"""Module tree of the Qwen2.5-VL vision tower on the MI355X kernels.

Class names, sub-module names, parameter shapes, construction order (hence default initialisation under a
given seed) and the ``forward(hidden_states, grid_thw)`` contract follow the reference's
python/models/qwen2_5_vl/modeling_qwen2_5_vl.py:192-262 and :324-1070; the arithmetic is done by
libmi355vit.so through ``mi355_vit.functional``.  The modules only run on a GPU: there is no CPU path.
"""

from __future__ import annotations

from collections import OrderedDict
from typing import Optional, Tuple

import torch
from torch import nn

from . import ops
from .config import Qwen2_5_VLVisionConfig
from .functional import (
    BLOCK_PARAM_ORDER,
    AttnGeometry,
    MergerFn,
    PatchEmbedFn,
    PatchEmbedFramesFn,
    PermuteRowsFn,
    VisionBlockFn,
    pack_block_weights,
)


class Qwen2RMSNorm(nn.Module):
    """Parameter holder for an RMSNorm (weight initialised to 1); the arithmetic is fused into its consumers."""

    def __init__(self, hidden_size: int, eps: float = 1e-6) -> None:
        super().__init__()
        self.weight = nn.Parameter(torch.ones(hidden_size))
        self.variance_epsilon = eps

    def extra_repr(self) -> str:
        return f"{tuple(self.weight.shape)}, eps={self.variance_epsilon}"


class Qwen2_5_VLMLP(nn.Module):
    def __init__(self, config, bias: bool = False) -> None:
        super().__init__()
        self.hidden_size = config.hidden_size
        self.intermediate_size = config.intermediate_size
        self.gate_proj = nn.Linear(self.hidden_size, self.intermediate_size, bias=bias)
        self.up_proj = nn.Linear(self.hidden_size, self.intermediate_size, bias=bias)
        self.down_proj = nn.Linear(self.intermediate_size, self.hidden_size, bias=bias)


class Qwen2_5_VisionPatchEmbed(nn.Module):
    def __init__(self, patch_size: int = 14, temporal_patch_size: int = 2, in_channels: int = 3, embed_dim: int = 1152) -> None:
        super().__init__()
        self.patch_size = patch_size
        self.temporal_patch_size = temporal_patch_size
        self.in_channels = in_channels
        self.embed_dim = embed_dim
        kernel_size = [temporal_patch_size, patch_size, patch_size]
        self.proj = nn.Conv3d(in_channels, embed_dim, kernel_size=kernel_size, stride=kernel_size, bias=False)

    def forward(self, hidden_states: torch.Tensor, compute_dtype: Optional[torch.dtype] = None) -> torch.Tensor:
        return PatchEmbedFn.apply(hidden_states, self.proj.weight, compute_dtype or self.proj.weight.dtype)

    fuse_frames = True  # bf16: make the rows of pixel_values inside the GEMM instead of writing them first

    def forward_frames(self, frames, compute_dtype: Optional[torch.dtype] = None) -> Tuple[torch.Tensor, torch.Tensor]:
        """Decoded, resized uint8 frame stacks (``[frames, H, W, 3]`` per image or video, on the GPU) -> (patch
        embeddings, ``image_grid_thw``): the image processor's rescale / normalise / patchify and this module's
        projection in one step."""
        from . import _lib, pixels

        T = compute_dtype or self.proj.weight.dtype
        frames = list(frames)
        if self.fuse_frames and T == torch.bfloat16 and pixels.frames_fit_fused_patch_embed(frames):
            try:
                return PatchEmbedFramesFn.apply(self.proj.weight, T, *frames), pixels.grid_thw_of(frames)
            except _lib.Unsupported:  # normalisation constants that do not fold into one multiply-add per byte
                pass
        rows, grid = pixels.patchify(frames, dtype=T)
        return self.forward(rows, T), grid


class Qwen2_5_VisionRotaryEmbedding(nn.Module):
    inv_freq: torch.Tensor

    def __init__(self, dim: int, theta: float = 10000.0) -> None:
        super().__init__()
        inv_freq = 1.0 / (theta ** (torch.arange(0, dim, 2, dtype=torch.float) / dim))
        self.register_buffer("inv_freq", inv_freq, persistent=False)

    def forward(self, seqlen: int) -> torch.Tensor:
        # arithmetic dtype follows the buffer (bf16 after model.to(bfloat16)), as in the reference (:242-245)
        seq = torch.arange(seqlen, device=self.inv_freq.device, dtype=self.inv_freq.dtype)
        return torch.outer(seq, self.inv_freq)


class Qwen2_5_VLPatchMerger(nn.Module):
    def __init__(self, dim: int, context_dim: int, spatial_merge_size: int = 2) -> None:
        super().__init__()
        self.hidden_size = context_dim * (spatial_merge_size**2)
        self.spatial_merge_unit = spatial_merge_size**2
        self.ln_q = Qwen2RMSNorm(context_dim, eps=1e-6)
        self.mlp = nn.Sequential(
            nn.Linear(self.hidden_size, self.hidden_size),
            nn.GELU(),
            nn.Linear(self.hidden_size, dim),
        )

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        return MergerFn.apply(x, self.ln_q.weight, self.mlp[0].weight, self.mlp[0].bias, self.mlp[2].weight, self.mlp[2].bias,
                              self.spatial_merge_unit, self.ln_q.variance_epsilon)


class Qwen2_5_VLVisionAttention(nn.Module):
    def __init__(self, config: Qwen2_5_VLVisionConfig, layer_index: int) -> None:
        super().__init__()
        self.dim = config.hidden_size
        self.num_heads = config.num_heads
        self.head_dim = self.dim // self.num_heads
        self.q_proj = nn.Linear(self.dim, self.dim, bias=True)
        self.k_proj = nn.Linear(self.dim, self.dim, bias=True)
        self.v_proj = nn.Linear(self.dim, self.dim, bias=True)
        self.proj = nn.Linear(self.dim, self.dim)
        self.scaling = self.head_dim**-0.5
        self.config = config
        self.attention_dropout = 0.0
        self.is_causal = False
        self.layer_index = layer_index
        self.fullatt_block = layer_index in config.fullatt_block_indexes


class Qwen2_5_VLVisionBlock(nn.Module):
    def __init__(self, config, layer_index: int, attn_implementation: str = "mi355_flash") -> None:
        super().__init__()
        self.norm1 = Qwen2RMSNorm(config.hidden_size, eps=1e-6)
        self.norm2 = Qwen2RMSNorm(config.hidden_size, eps=1e-6)
        self.attn = Qwen2_5_VLVisionAttention(config=config, layer_index=layer_index)
        self.mlp = Qwen2_5_VLMLP(config, bias=True)
        self.gradient_checkpointing = False
        self._packed = None
        self._packed_key = None

    def _block_params(self):
        """The 16 parameters in BLOCK_PARAM_ORDER, read from the module dictionaries directly: this runs three times per
        block and step, and 48 `get_parameter` calls per block cost more host time than the block's launches."""
        m = self._modules
        at, ml = m["attn"]._modules, m["mlp"]._modules
        q, k, v, pr = at["q_proj"]._parameters, at["k_proj"]._parameters, at["v_proj"]._parameters, at["proj"]._parameters
        g, u, d = ml["gate_proj"]._parameters, ml["up_proj"]._parameters, ml["down_proj"]._parameters
        return [m["norm1"]._parameters["weight"], m["norm2"]._parameters["weight"],
                q["weight"], q["bias"], k["weight"], k["bias"], v["weight"], v["bias"], pr["weight"], pr["bias"],
                g["weight"], g["bias"], u["weight"], u["bias"], d["weight"], d["bias"]]

    def packed(self, dtype: torch.dtype):
        """Packed compute-dtype operands.  They are rebuilt when a parameter was replaced or modified in place
        through torch (load_state_dict, a torch optimizer: the version counter moves); FusedAdam updates parameters
        through raw pointers and writes the packed copies itself in the same pass, so its steps need no rebuild."""
        params = self._block_params()
        key = (dtype,) + tuple((p.data_ptr(), p._version) for p in params)
        if key != self._packed_key:
            self._packed = pack_block_weights(params, dtype, self._packed)
            self._packed_key = key
        return self._packed

    def forward(
        self,
        hidden_states: torch.Tensor,
        cu_seqlens: torch.Tensor,
        rotary_pos_emb: Optional[torch.Tensor] = None,
        position_embeddings: Optional[Tuple[torch.Tensor, torch.Tensor]] = None,
        **kwargs,
    ) -> torch.Tensor:
        geo = kwargs.get("_geometry")
        if geo is None:
            if position_embeddings is None:
                emb = torch.cat((rotary_pos_emb, rotary_pos_emb), dim=-1)
                position_embeddings = (emb.cos(), emb.sin())
            cu_host = cu_seqlens.detach().cpu()  # host sync, as in the reference (:433)
            lengths = cu_host[1:] - cu_host[:-1]
            max_seqlen = int(lengths.max()) if lengths.numel() else 0
            order = ops.segment_order(lengths)
            ops.check_segments(cu_host, hidden_states.shape[0], max_seqlen, order)
            geo = AttnGeometry(
                cu_seqlens.to(device=hidden_states.device, dtype=torch.int32).contiguous(), max_seqlen,
                self.attn.num_heads, self.attn.head_dim,
                position_embeddings[0].float().contiguous(), position_embeddings[1].float().contiguous(),
                None if order is None else order.to(hidden_states.device),
            )
        ckpt = self.gradient_checkpointing and self.training and torch.is_grad_enabled()
        return VisionBlockFn.apply(hidden_states, self, geo, self.norm1.variance_epsilon, ckpt, *self._block_params())


class _TowerPlan:
    """Host-side plan of one forward: permutations, segment boundaries and rotary tables for a grid_thw."""

    def __init__(self, model: "Qwen2_5_VisionTransformerPretrainedModel", grid: torch.Tensor, device: torch.device):
        merge = model.spatial_merge_size
        unit = model.spatial_merge_unit
        self.window_index_cpu, cu_w = ops.window_index(grid, merge, model.window_size, model.patch_size)
        self.reverse_index_cpu = torch.empty_like(self.window_index_cpu)
        self.reverse_index_cpu[self.window_index_cpu] = torch.arange(self.window_index_cpu.numel())
        cu_f = ops.cu_seqlens(grid)
        pos = ops.rot_pos_ids(grid, merge)
        S = pos.shape[0]
        self.seq_len = S
        # rotary angles are gathered straight into window order (permute the ids, not the table)
        pos = pos.view(S // unit, unit, 2)[self.window_index_cpu].reshape(S, 2)
        self.pos_ids = pos.to(device)
        self.max_grid = int(grid[:, 1:].max())
        self.window_index = self.window_index_cpu.to(device)
        self.reverse_index = self.reverse_index_cpu.to(device)
        self.cu_window_cpu, self.cu_full_cpu = cu_w, cu_f
        self.cu_window, self.cu_full = cu_w.to(device), cu_f.to(device)
        self.max_window = int((cu_w[1:] - cu_w[:-1]).max()) if cu_w.numel() > 1 else 0
        self.max_full = int((cu_f[1:] - cu_f[:-1]).max()) if cu_f.numel() > 1 else 0
        order_w, order_f = ops.segment_order(cu_w[1:] - cu_w[:-1]), ops.segment_order(cu_f[1:] - cu_f[:-1])
        ops.check_segments(cu_w, S, self.max_window, order_w)
        ops.check_segments(cu_f, S, self.max_full, order_f)
        self.order_window = None if order_w is None else order_w.to(device)
        self.order_full = None if order_f is None else order_f.to(device)


class Qwen2_5_VisionTransformerPretrainedModel(nn.Module):
    """Drop-in for the reference class of the same name (modeling:809-1070), non-sequence-parallel branch."""

    def __init__(self, config: Qwen2_5_VLVisionConfig, *inputs, **kwargs) -> None:
        super().__init__()
        self.config = config
        self.spatial_merge_size = config.spatial_merge_size
        self.patch_size = config.patch_size
        self.fullatt_block_indexes = config.fullatt_block_indexes
        self.window_size = config.window_size
        self.spatial_merge_unit = self.spatial_merge_size * self.spatial_merge_size

        self.patch_embed = Qwen2_5_VisionPatchEmbed(
            patch_size=config.patch_size,
            temporal_patch_size=config.temporal_patch_size,
            in_channels=config.in_channels,
            embed_dim=config.hidden_size,
        )
        head_dim = config.hidden_size // config.num_heads
        self.rotary_pos_emb = Qwen2_5_VisionRotaryEmbedding(head_dim // 2)
        self.blocks = nn.ModuleList([Qwen2_5_VLVisionBlock(config, i) for i in range(config.depth)])
        self.merger = Qwen2_5_VLPatchMerger(
            dim=config.out_hidden_size,
            context_dim=config.hidden_size,
            spatial_merge_size=config.spatial_merge_size,
        )
        self.gradient_checkpointing = False
        self.sequence_parallel = config.sequence_parallel
        self._plans: "OrderedDict[tuple, _TowerPlan]" = OrderedDict()

    # ---- reference-compatible helpers -----------------------------------------------------------
    def gradient_checkpointing_enable(self, gradient_checkpointing_kwargs=None) -> None:
        self.gradient_checkpointing = True
        for blk in self.blocks:
            blk.gradient_checkpointing = True

    def gradient_checkpointing_disable(self) -> None:
        self.gradient_checkpointing = False
        for blk in self.blocks:
            blk.gradient_checkpointing = False

    @property
    def dtype(self) -> torch.dtype:
        return self.patch_embed.proj.weight.dtype

    @property
    def device(self) -> torch.device:
        return self.patch_embed.proj.weight.device

    def rot_pos_emb(self, grid_thw: torch.Tensor) -> torch.Tensor:
        """[S, head_dim/2] angle table in patch order (modeling:841-868)."""
        pos_ids = ops.rot_pos_ids(grid_thw, self.spatial_merge_size).to(self.rotary_pos_emb.inv_freq.device)
        full = self.rotary_pos_emb(int(grid_thw[:, 1:].max()))
        return full[pos_ids].flatten(1)

    def get_window_index(self, grid_thw: torch.Tensor):
        """(window_index int64 tensor, cu_window_seqlens list) as modeling:870-909, already free of repeated entries."""
        idx, cu = ops.window_index(grid_thw, self.spatial_merge_size, self.window_size, self.patch_size)
        return idx.to(grid_thw.device), cu.tolist()

    def _plan(self, grid_thw: torch.Tensor, device: torch.device, host: Optional[torch.Tensor] = None) -> _TowerPlan:
        # the plan needs the grid on the host: a copy the caller still holds there (grids are born on the host, in the
        # data pipeline) saves the device -> host read, which would make the host wait for all GPU work issued so far
        grid = (host if host is not None else grid_thw).detach().to("cpu", torch.int64).reshape(-1, 3)
        if host is not None and tuple(grid.shape) != tuple(grid_thw.reshape(-1, 3).shape):
            raise ValueError(f"grid_thw_host {tuple(host.shape)} does not have the shape of grid_thw {tuple(grid_thw.shape)}")
        key = (tuple(grid.flatten().tolist()), str(device))
        plan = self._plans.get(key)
        if plan is None:
            plan = _TowerPlan(self, grid, device)
            self._plans[key] = plan
            while len(self._plans) > 16:
                self._plans.popitem(last=False)
        else:
            self._plans.move_to_end(key)
        return plan

    def _compute_dtype(self) -> torch.dtype:
        if torch.is_autocast_enabled("cuda"):
            return torch.get_autocast_dtype("cuda")
        return self.dtype

    # ---- forward ---------------------------------------------------------------------------------
    def forward(self, hidden_states: Optional[torch.Tensor] = None, grid_thw: Optional[torch.Tensor] = None, *, frames=None,
                grid_thw_host: Optional[torch.Tensor] = None, **kwargs) -> torch.Tensor:
        """hidden_states: pixels view-able to [-1, in_channels*temporal_patch*patch*patch]; grid_thw [N,3] int64.
        Returns [S / merge^2, out_hidden_size] in the original (un-windowed) token order.
        ``grid_thw_host`` (optional): the same values in a CPU tensor; a grid on the GPU is otherwise read back, which
        makes the host wait for the GPU (the reference reads it back with ``.tolist()``, modeling:848, :876).
        ``frames`` (instead of ``hidden_states``; ``grid_thw`` then follows from their shapes): decoded, resized uint8
        frame stacks ``[frames, H, W, 3]`` on the GPU, one per image or video."""
        if self.sequence_parallel:
            raise NotImplementedError(
                "sequence_parallel=True needs inter-GPU collectives, which this single-GPU build does not have; "
                "use mi355_vit.sequence_parallel_utils for the per-rank pack/unpack and run the tower unsharded."
            )
        device = self.device
        if device.type != "cuda":
            raise RuntimeError("the MI355X vision tower runs on the GPU only (move the module with .to('cuda'))")
        T = self._compute_dtype()
        if T not in (torch.float32, torch.bfloat16):
            raise TypeError(f"compute dtype {T} is not supported (float32 or bfloat16)")
        if (hidden_states is None) == (frames is None):
            raise ValueError("pass either hidden_states (with grid_thw) or frames")
        if frames is not None:
            x, grid_of_frames = self.patch_embed.forward_frames(frames, T)
            if grid_thw is not None and grid_thw.detach().to("cpu", torch.int64).reshape(-1, 3).tolist() != grid_of_frames.tolist():
                raise ValueError(f"grid_thw {grid_thw.tolist()} does not describe the frames ({grid_of_frames.tolist()})")
            grid_thw = grid_of_frames
        elif grid_thw is None:
            raise ValueError("hidden_states needs grid_thw")
        plan = self._plan(grid_thw, device, grid_thw_host if frames is None else None)
        unit = self.spatial_merge_unit

        if frames is None:
            x = self.patch_embed(hidden_states.to(device), T)
        if x.shape[0] != plan.seq_len:
            raise ValueError(f"hidden_states holds {x.shape[0]} patches but grid_thw describes {plan.seq_len}")
        x = PermuteRowsFn.apply(x, plan.window_index, plan.reverse_index, unit)

        # rotary tables: same torch ops and dtype propagation as the reference (:866-867, :941-942, :278)
        table = self.rotary_pos_emb(plan.max_grid)[plan.pos_ids].flatten(1)
        emb = torch.cat((table, table), dim=-1)
        cos, sin = emb.cos().float().contiguous(), emb.sin().float().contiguous()

        H, hd = self.config.num_heads, self.config.hidden_size // self.config.num_heads
        geo_full = AttnGeometry(plan.cu_full, plan.max_full, H, hd, cos, sin, plan.order_full)
        geo_win = AttnGeometry(plan.cu_window, plan.max_window, H, hd, cos, sin, plan.order_window)
        for layer_num, blk in enumerate(self.blocks):
            full = layer_num in self.fullatt_block_indexes
            x = blk(x, cu_seqlens=plan.cu_full if full else plan.cu_window, position_embeddings=(cos, sin),
                    _geometry=geo_full if full else geo_win)

        x = self.merger(x)
        return PermuteRowsFn.apply(x, plan.reverse_index, plan.window_index, 1)
