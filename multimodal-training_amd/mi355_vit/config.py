"""Plain configuration object with the field names of the reference's Qwen2_5_VLVisionConfig
(python/models/qwen2_5_vl/configuration_qwen2_5_vl.py:32-71)."""

from __future__ import annotations

from dataclasses import asdict, dataclass, field
from typing import List


@dataclass
class Qwen2_5_VLVisionConfig:
    depth: int = 32
    hidden_size: int = 3584  # the reference's class default; the real tower uses 1280
    hidden_act: str = "silu"
    intermediate_size: int = 3420
    num_heads: int = 16
    in_channels: int = 3
    patch_size: int = 14
    spatial_merge_size: int = 2
    temporal_patch_size: int = 2
    tokens_per_second: int = 4
    window_size: int = 112
    out_hidden_size: int = 3584
    fullatt_block_indexes: List[int] = field(default_factory=lambda: [7, 15, 23, 31])
    initializer_range: float = 0.02
    sequence_parallel: bool = False
    _attn_implementation: str = "mi355_flash"

    model_type = "qwen2_5_vl"

    def __post_init__(self) -> None:
        if self.hidden_act != "silu":
            raise ValueError(f"hidden_act={self.hidden_act!r}: only 'silu' is implemented")
        if self.hidden_size % self.num_heads:
            raise ValueError("hidden_size must be a multiple of num_heads")

    def to_dict(self) -> dict:
        return asdict(self)

    @classmethod
    def qwen2_5_vl_tower(cls, **overrides) -> "Qwen2_5_VLVisionConfig":
        """The 675 M-parameter tower: depth 32, hidden 1280, 16 heads of 80, SwiGLU 3420, merger to 3584."""
        base = dict(depth=32, hidden_size=1280, intermediate_size=3420, num_heads=16, out_hidden_size=3584)
        base.update(overrides)
        return cls(**base)
