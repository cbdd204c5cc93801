"""Input side on the GPU: decoded, resized RGB frames -> ``pixel_values`` and ``image_grid_thw``.

The reference produces these two tensors on CPU dataloader workers: ``python/data/preprocessing.py:134`` calls
``processor.apply_chat_template``, whose image processor (transformers 4.57.0, ``Qwen2VLImageProcessor``)
rescales, normalises and cuts every image into ``[grid_t * grid_h * grid_w, 1176]`` rows, and
``python/data/collator.py:134-156`` concatenates the samples.  ``patchify`` does the same for frames that are
already on the GPU as uint8 ``[frames, height, width, 3]`` (height and width multiples of 28, i.e. after the
processor's resize step, which stays where the frames are decoded), for the whole batch in one launch, with the
processor's arithmetic (float32 results are bit-identical to a numpy restatement of it) and, optionally, the cast
to the model dtype that the tower applies first.

There is no CPU path: frames must live on the GPU and the HIP library must be built.
"""

from __future__ import annotations

import ctypes as C
from typing import Optional, Sequence, Tuple

import numpy as np
import torch

from . import _lib

OPENAI_CLIP_MEAN = (0.48145466, 0.4578275, 0.40821073)
OPENAI_CLIP_STD = (0.26862954, 0.26130258, 0.27577711)
PATCH_SIZE, TEMPORAL_PATCH_SIZE, MERGE_SIZE = 14, 2, 2

_TABLE_DTYPE = np.dtype([("pixels", "<u8"), ("frames", "<i4"), ("height", "<i4"), ("width", "<i4"), ("reserved", "<i4"),
                         ("first_row", "<i8")])
assert _TABLE_DTYPE.itemsize == C.sizeof(_lib.Image) == 32


def grid_thw_of(frames: Sequence[torch.Tensor]) -> torch.Tensor:
    """``image_grid_thw`` ([n, 3] int64, CPU) of resized frame stacks, as the processor reports it."""
    rows = []
    for i, f in enumerate(frames):
        if f.dim() != 4 or f.shape[3] != 3 or f.dtype != torch.uint8:
            raise ValueError(f"image {i}: expected uint8 [frames, height, width, 3], got {f.dtype} {tuple(f.shape)}")
        n, h, w, _ = f.shape
        unit = PATCH_SIZE * MERGE_SIZE
        if n < 1 or h < unit or w < unit or h % unit or w % unit:
            raise ValueError(f"image {i}: {n} frames of {h}x{w}; height and width must be multiples of {unit} "
                             "(run the processor's resize first)")
        rows.append(((n + TEMPORAL_PATCH_SIZE - 1) // TEMPORAL_PATCH_SIZE, h // PATCH_SIZE, w // PATCH_SIZE))
    return torch.tensor(rows, dtype=torch.int64).reshape(-1, 3)


def patchify(frames: Sequence[torch.Tensor], dtype: torch.dtype = torch.float32,
             image_mean: Sequence[float] = OPENAI_CLIP_MEAN, image_std: Sequence[float] = OPENAI_CLIP_STD,
             rescale_factor: float = 1.0 / 255.0, out: Optional[torch.Tensor] = None) -> Tuple[torch.Tensor, torch.Tensor]:
    """Frames of a batch of images / videos -> (``pixel_values`` [rows, 1176] on the GPU, ``image_grid_thw`` [n, 3]).

    ``frames``: one contiguous uint8 GPU tensor ``[frames, height, width, 3]`` per image (one frame) or video.
    ``dtype``: float32 (what the processor returns) or bfloat16 (what the tower casts it to).
    """
    frames = list(frames)
    if not frames:
        raise ValueError("patchify: no images")
    grid = grid_thw_of(frames)
    device = frames[0].device
    for i, f in enumerate(frames):
        if not f.is_cuda or f.device != device:
            raise RuntimeError(f"image {i} on {f.device}: frames must be on one GPU (there is no CPU path)")
        if not f.is_contiguous():
            raise RuntimeError(f"image {i}: frames must be contiguous")
    if dtype == torch.float32:
        code = _lib.F32
    elif dtype == torch.bfloat16:
        code = _lib.BF16
    else:
        raise TypeError(f"unsupported dtype {dtype} (float32 and bfloat16 only)")
    counts = (grid[:, 0] * grid[:, 1] * grid[:, 2]).numpy()
    n = len(frames)
    table = np.zeros(n + 1, dtype=_TABLE_DTYPE)
    table["pixels"][:n] = [f.data_ptr() for f in frames]
    table["frames"][:n] = [f.shape[0] for f in frames]
    table["height"][:n] = [f.shape[1] for f in frames]
    table["width"][:n] = [f.shape[2] for f in frames]
    table["first_row"][1:] = np.cumsum(counts)
    total = int(table["first_row"][n])
    if out is None:
        out = torch.empty((total, _lib.PIXEL_ROW), dtype=dtype, device=device)
    elif out.shape != (total, _lib.PIXEL_ROW) or out.dtype != dtype or out.device != device or not out.is_contiguous():
        raise RuntimeError(f"patchify: out must be a contiguous {dtype} [{total}, {_lib.PIXEL_ROW}] tensor on {device}")
    dev_table = torch.from_numpy(table.view(np.uint8)).to(device)  # 32 bytes per image, synchronous copy
    mean = [float(np.float32(m)) for m in image_mean]
    std = [float(np.float32(s)) for s in image_std]
    lib = _lib.load()
    with torch.cuda.device(device):
        stream = torch.cuda.current_stream(device).cuda_stream
        rc = lib.mvit_patchify(dev_table.data_ptr(), n, total, out.data_ptr(), float(rescale_factor), *mean, *std, code, stream)
    _lib.check(rc, "mvit_patchify")
    return out, grid
