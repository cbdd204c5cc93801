"""Input side on the GPU: decoded RGB frames -> (resize ->) ``pixel_values`` and ``image_grid_thw``.

The reference produces these two tensors on CPU dataloader workers: ``python/data/preprocessing.py:134`` calls
``processor.apply_chat_template``, whose image processor (transformers 4.57.0, ``Qwen2VLImageProcessor``)
rescales, normalises and cuts every image into ``[grid_t * grid_h * grid_w, 1176]`` rows, and
``python/data/collator.py:134-156`` concatenates the samples.  ``patchify`` does the same for frames that are
already on the GPU as uint8 ``[frames, height, width, 3]`` (height and width multiples of 28, i.e. after the
processor's resize step, which stays where the frames are decoded), for the whole batch in one launch, with the
processor's arithmetic (float32 results are bit-identical to a numpy restatement of it) and, optionally, the cast
to the model dtype that the tower applies first.

``resize_frames`` is the step in front of it: ``PIL.Image.resize`` for 8-bit RGB frames (BILINEAR: the reference's own
fixed-size resize, ``python/data/preprocessing.py:126-131``; BICUBIC: the image processor's resize to the
``smart_resize`` target), bit for bit, as two resampling passes on the GPU; the coefficient tables are computed on the
host exactly as Pillow computes them.  ``preprocess`` chains smart_resize -> resize -> patchify for still images.

There is no CPU path: frames must live on the GPU and the HIP library must be built.
"""

from __future__ import annotations

import ctypes as C
import functools
import math
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


def _image_table(frames: Sequence[torch.Tensor], what: str):
    """Checks the frame stacks and builds the device table of ``mvit_image`` entries (32 bytes per image, one
    synchronous copy).  Returns (frames as a list, image_grid_thw, device table, total rows)."""
    frames = list(frames)
    if not frames:
        raise ValueError(f"{what}: no images")
    grid = grid_thw_of(frames)
    device = frames[0].device
    for i, f in enumerate(frames):
        if not f.is_cuda or f.device != device:
            raise RuntimeError(f"image {i} on {f.device}: frames must be on one GPU (there is no CPU path)")
        if not f.is_contiguous():
            raise RuntimeError(f"image {i}: frames must be contiguous")
    counts = (grid[:, 0] * grid[:, 1] * grid[:, 2]).numpy()
    n = len(frames)
    table = np.zeros(n + 1, dtype=_TABLE_DTYPE)
    table["pixels"][:n] = [f.data_ptr() for f in frames]
    table["frames"][:n] = [f.shape[0] for f in frames]
    table["height"][:n] = [f.shape[1] for f in frames]
    table["width"][:n] = [f.shape[2] for f in frames]
    table["first_row"][1:] = np.cumsum(counts)
    total = int(table["first_row"][n])
    return frames, grid, torch.from_numpy(table.view(np.uint8)).to(device), total


def patchify(frames: Sequence[torch.Tensor], dtype: torch.dtype = torch.float32,
             image_mean: Sequence[float] = OPENAI_CLIP_MEAN, image_std: Sequence[float] = OPENAI_CLIP_STD,
             rescale_factor: float = 1.0 / 255.0, out: Optional[torch.Tensor] = None) -> Tuple[torch.Tensor, torch.Tensor]:
    """Frames of a batch of images / videos -> (``pixel_values`` [rows, 1176] on the GPU, ``image_grid_thw`` [n, 3]).

    ``frames``: one contiguous uint8 GPU tensor ``[frames, height, width, 3]`` per image (one frame) or video.
    ``dtype``: float32 (what the processor returns) or bfloat16 (what the tower casts it to).
    """
    if dtype == torch.float32:
        code = _lib.F32
    elif dtype == torch.bfloat16:
        code = _lib.BF16
    else:
        raise TypeError(f"unsupported dtype {dtype} (float32 and bfloat16 only)")
    frames, grid, dev_table, total = _image_table(frames, "patchify")
    n, device = len(frames), frames[0].device
    if out is None:
        out = torch.empty((total, _lib.PIXEL_ROW), dtype=dtype, device=device)
    elif out.shape != (total, _lib.PIXEL_ROW) or out.dtype != dtype or out.device != device or not out.is_contiguous():
        raise RuntimeError(f"patchify: out must be a contiguous {dtype} [{total}, {_lib.PIXEL_ROW}] tensor on {device}")
    mean = [float(np.float32(m)) for m in image_mean]
    std = [float(np.float32(s)) for s in image_std]
    lib = _lib.load()
    with torch.cuda.device(device):
        stream = torch.cuda.current_stream(device).cuda_stream
        rc = lib.mvit_patchify(dev_table.data_ptr(), n, total, out.data_ptr(), float(rescale_factor), *mean, *std, code, stream)
    _lib.check(rc, "mvit_patchify")
    return out, grid


PACKED_PATCH_K = 1344  # 28 pixel lines of a patch (frame of the pair, y), each 14 x 3 bytes padded to 48


def frames_fit_fused_patch_embed(frames: Sequence[torch.Tensor]) -> bool:
    """Whether ``patch_embed_frames`` can read these frame stacks: 4-byte aligned buffers below 2 GiB each."""
    return all(f.data_ptr() % 4 == 0 and f.numel() < 2**31 for f in frames)


def pack_patch_embed_weight(weight: torch.Tensor) -> torch.Tensor:
    """The patch-embedding weight ([embed_dim, 1176] or the Conv3d's [embed_dim, 3, 2, 14, 14], float32 or bfloat16)
    in the contraction order of ``patch_embed_frames``: bfloat16 ``[embed_dim, 1344]``."""
    w = weight.detach().reshape(weight.shape[0], -1)
    if w.shape[1] != _lib.PIXEL_ROW or w.dtype not in (torch.float32, torch.bfloat16) or not w.is_cuda:
        raise ValueError(f"pack_patch_embed_weight: expected a float32 / bfloat16 GPU weight with {_lib.PIXEL_ROW} inputs, got {w.dtype} {tuple(w.shape)} on {w.device}")
    if w.stride(1) != 1:
        w = w.contiguous()
    packed = torch.empty((w.shape[0], PACKED_PATCH_K), dtype=torch.bfloat16, device=w.device)
    lib = _lib.load()
    with torch.cuda.device(w.device):
        rc = lib.mvit_patch_embed_pack_weight(w.data_ptr(), _lib.BF16 if w.dtype == torch.bfloat16 else _lib.F32, w.stride(0),
                                              w.shape[0], packed.data_ptr(), torch.cuda.current_stream(w.device).cuda_stream)
    _lib.check(rc, "mvit_patch_embed_pack_weight")
    return packed


def patch_embed_frames(frames: Sequence[torch.Tensor], packed_weight: torch.Tensor, dtype: torch.dtype = torch.bfloat16,
                       image_mean: Sequence[float] = OPENAI_CLIP_MEAN, image_std: Sequence[float] = OPENAI_CLIP_STD,
                       rescale_factor: float = 1.0 / 255.0) -> Tuple[torch.Tensor, torch.Tensor]:
    """Frames -> (patch embeddings ``[rows, embed_dim]``, ``image_grid_thw``): ``patchify(frames, bfloat16)`` times the
    weight, in one kernel that makes the rows on the fly and never writes them.  ``packed_weight`` comes from
    ``pack_patch_embed_weight``.  Raises ``_lib.Unsupported`` when the normalisation constants cannot be folded into
    one multiply-add per byte without changing a bfloat16 value (the caller then uses ``patchify`` and a GEMM)."""
    if dtype not in (torch.float32, torch.bfloat16):
        raise TypeError(f"unsupported dtype {dtype} (float32 and bfloat16 only)")
    frames, grid, dev_table, total = _image_table(frames, "patch_embed_frames")
    device = frames[0].device
    if not frames_fit_fused_patch_embed(frames):
        raise RuntimeError("patch_embed_frames: frame buffers must be 4-byte aligned and smaller than 2 GiB")
    if (packed_weight.dim() != 2 or packed_weight.shape[1] != PACKED_PATCH_K or packed_weight.dtype != torch.bfloat16
            or packed_weight.device != device or not packed_weight.is_contiguous()):
        raise ValueError("patch_embed_frames: packed_weight must be the contiguous bfloat16 [embed_dim, 1344] result of pack_patch_embed_weight on the frames' GPU")
    out = torch.empty((total, packed_weight.shape[0]), dtype=dtype, device=device)
    mean = [float(np.float32(m)) for m in image_mean]
    std = [float(np.float32(s)) for s in image_std]
    lib = _lib.load()
    with torch.cuda.device(device):
        rc = lib.mvit_patch_embed_frames(dev_table.data_ptr(), len(frames), total, packed_weight.data_ptr(), packed_weight.shape[0],
                                         out.data_ptr(), out.stride(0), _lib.BF16 if dtype == torch.bfloat16 else _lib.F32,
                                         float(rescale_factor), *mean, *std, torch.cuda.current_stream(device).cuda_stream)
    _lib.check(rc, "mvit_patch_embed_frames")
    return out, grid


# ------------------------------------------------------------------------------------------------ resize

BILINEAR, BICUBIC = "bilinear", "bicubic"
_FILTER_SUPPORT = {BILINEAR: 1.0, BICUBIC: 2.0}
_PRECISION_BITS = 22  # Pillow: 32 - 8 bits of pixel - 2 bits of head-room


def smart_resize(height: int, width: int, factor: int = PATCH_SIZE * MERGE_SIZE, min_pixels: int = 56 * 56,
                 max_pixels: int = 14 * 14 * 4 * 1280) -> Tuple[int, int]:
    """The (height, width) the image processor resizes to (transformers 4.57.0 ``smart_resize``): multiples of
    ``factor``, pixel count within [min_pixels, max_pixels], aspect ratio kept as closely as that allows."""
    if height <= 0 or width <= 0:
        raise ValueError(f"smart_resize: {height}x{width}")
    if max(height, width) / min(height, width) > 200:
        raise ValueError(f"absolute aspect ratio must be smaller than 200, got {max(height, width) / min(height, width)}")
    h_bar = round(height / factor) * factor
    w_bar = round(width / factor) * factor
    if h_bar * w_bar > max_pixels:
        beta = math.sqrt((height * width) / max_pixels)
        h_bar = max(factor, math.floor(height / beta / factor) * factor)
        w_bar = max(factor, math.floor(width / beta / factor) * factor)
    elif h_bar * w_bar < min_pixels:
        beta = math.sqrt(min_pixels / (height * width))
        h_bar = math.ceil(height * beta / factor) * factor
        w_bar = math.ceil(width * beta / factor) * factor
    return h_bar, w_bar


def resample_coefficients(in_size: int, out_size: int, resample: str = BICUBIC) -> Tuple[np.ndarray, np.ndarray]:
    """Window bounds ([out_size, 2] int32: first input index, tap count) and 22-bit fixed-point weights ([out_size, ksize]
    int32) of one axis, as Pillow's Resample.c computes them (precompute_coeffs + normalize_coeffs_8bpc): the filter's
    support is widened by the scale factor when shrinking; weights are evaluated and normalised in double precision, the
    sum taken tap by tap in index order.  Every step is one IEEE double operation, in the order of the C source, so the
    tables are Pillow's bit for bit."""
    if resample not in _FILTER_SUPPORT:
        raise ValueError(f"resample must be '{BILINEAR}' or '{BICUBIC}', got {resample!r}")
    if in_size < 1 or out_size < 1:
        raise ValueError(f"resample_coefficients: sizes {in_size} -> {out_size}")
    scale = in_size / out_size
    filterscale = scale if scale >= 1.0 else 1.0
    support = _FILTER_SUPPORT[resample] * filterscale
    ksize = int(math.ceil(support)) * 2 + 1
    ss = 1.0 / filterscale
    center = (np.arange(out_size, dtype=np.float64) + 0.5) * scale
    xmin = np.maximum((center - support + 0.5).astype(np.int64), 0)  # (int) truncates; the operand is > -1 here
    xmax = np.minimum((center + support + 0.5).astype(np.int64), in_size) - xmin
    taps = np.arange(ksize, dtype=np.int64)[None, :]
    active = taps < xmax[:, None]
    x = np.abs(((taps + xmin[:, None]).astype(np.float64) - center[:, None] + 0.5) * ss)
    if resample == BILINEAR:
        w = np.where(x < 1.0, 1.0 - x, 0.0)
    else:
        a = -0.5
        w = np.where(x < 1.0, ((a + 2.0) * x - (a + 3.0)) * x * x + 1, np.where(x < 2.0, (((x - 5) * x + 8) * x - 4) * a, 0.0))
    w = np.where(active, w, 0.0)
    ww = np.cumsum(w, axis=1)[:, -1:]  # left-to-right sum, like the C loop (numpy's sum() adds pairwise)
    w = np.where(ww != 0.0, w / np.where(ww != 0.0, ww, 1.0), w)
    fixed = np.where(w < 0, -0.5 + w * (1 << _PRECISION_BITS), 0.5 + w * (1 << _PRECISION_BITS)).astype(np.int64)  # truncation
    kk = np.where(active, fixed, 0).astype(np.int32)
    bounds = np.stack([xmin, xmax], axis=1).astype(np.int32)
    return bounds, kk


@functools.lru_cache(maxsize=64)
def _device_coefficients(in_size: int, out_size: int, resample: str, device_index: int):
    bounds, kk = resample_coefficients(in_size, out_size, resample)
    dev = torch.device("cuda", device_index)
    return torch.from_numpy(bounds).to(dev), torch.from_numpy(kk).to(dev), kk.shape[1]


def resize_frames(frames: torch.Tensor, out_height: int, out_width: int, resample: str = BICUBIC) -> torch.Tensor:
    """``PIL.Image.resize((out_width, out_height), resample)`` applied to every frame of a contiguous uint8 GPU tensor
    ``[frames, height, width, 3]``, bit for bit: a horizontal pass into an 8-bit intermediate image, then a vertical
    pass (a pass whose size does not change is skipped, as Pillow does)."""
    if frames.dim() != 4 or frames.dtype != torch.uint8 or frames.shape[0] < 1:
        raise ValueError(f"resize_frames: expected uint8 [frames, height, width, channels], got {frames.dtype} {tuple(frames.shape)}")
    if not frames.is_cuda:
        raise RuntimeError("resize_frames: frames must be on the GPU (there is no CPU path)")
    if not frames.is_contiguous():
        raise RuntimeError("resize_frames: frames must be contiguous")
    if out_height < 1 or out_width < 1:
        raise ValueError(f"resize_frames: target {out_height}x{out_width}")
    n, h, w, ch = frames.shape
    lib = _lib.load()
    device = frames.device
    cur = frames
    with torch.cuda.device(device):
        stream = torch.cuda.current_stream(device).cuda_stream
        if w != out_width:
            bounds, kk, ksize = _device_coefficients(w, out_width, resample, device.index or 0)
            nxt = torch.empty((n, h, out_width, ch), dtype=torch.uint8, device=device)
            _lib.check(lib.mvit_resample_u8(cur.data_ptr(), nxt.data_ptr(), n * h, w, out_width, ch, bounds.data_ptr(), kk.data_ptr(),
                                            ksize, stream), "mvit_resample_u8")
            cur = nxt
        if h != out_height:
            bounds, kk, ksize = _device_coefficients(h, out_height, resample, device.index or 0)
            nxt = torch.empty((n, out_height, out_width, ch), dtype=torch.uint8, device=device)
            _lib.check(lib.mvit_resample_u8(cur.data_ptr(), nxt.data_ptr(), n, h, out_height, out_width * ch, bounds.data_ptr(),
                                            kk.data_ptr(), ksize, stream), "mvit_resample_u8")
            cur = nxt
    return cur.clone() if cur is frames else cur


def preprocess(images: Sequence[torch.Tensor], dtype: torch.dtype = torch.float32, min_pixels: int = 56 * 56,
               max_pixels: int = 14 * 14 * 4 * 1280, resample: str = BICUBIC) -> Tuple[torch.Tensor, torch.Tensor]:
    """Decoded still images (uint8 GPU tensors ``[1, height, width, 3]`` of any size) -> (``pixel_values``,
    ``image_grid_thw``): the image processor's smart_resize + resize + rescale + normalise + patchify, on the GPU."""
    resized = []
    for i, f in enumerate(images):
        if f.dim() != 4 or f.shape[0] != 1 or f.shape[3] != 3:
            raise ValueError(f"image {i}: expected uint8 [1, height, width, 3], got {tuple(f.shape)}")
        th, tw = smart_resize(int(f.shape[1]), int(f.shape[2]), min_pixels=min_pixels, max_pixels=max_pixels)
        resized.append(resize_frames(f, th, tw, resample))
    return patchify(resized, dtype=dtype)
