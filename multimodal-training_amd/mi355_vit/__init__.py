"""mi355_vit -- MI355X-native Qwen2.5-VL vision tower (forward + backward) behind the reference's
VisionTrainer / vision-model interfaces.  Importing the package does not touch the GPU; the first kernel call
loads ``libmi355vit.so`` and raises if it has not been built."""

from .config import Qwen2_5_VLVisionConfig  # noqa: F401

__all__ = ["Qwen2_5_VLVisionConfig"]
