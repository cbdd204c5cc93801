"""CPU oracle of the resize step in front of the patch rows.  TEST INFRASTRUCTURE ONLY: imported by tests/ and the
smoke check, never by the product.

What it restates
  * ``smart_resize``: the target size the image processor picks (transformers 4.57.0,
    ``models/qwen2_vl/image_processing_qwen2_vl.py``; the reference reaches it through
    ``processor.apply_chat_template``, python/data/preprocessing.py:134): both sides multiples of 28, pixel count
    inside [min_pixels, max_pixels], aspect ratio kept as closely as that allows.
  * ``pil_resize``: ``PIL.Image.resize`` for 8-bit RGB images with the BILINEAR filter (the reference's own fixed-size
    resize, python/data/preprocessing.py:126-131) and the BICUBIC filter (the image processor's resample), as
    Pillow's libImaging/Resample.c computes it: filter support widened by the scale factor when shrinking,
    coefficients in double precision normalised to sum 1, converted to 22-bit fixed point, a horizontal pass into an
    8-bit intermediate image, then a vertical pass, each with rounding and clipping to 0..255.

Pins (tests/test_oracle_resize.py): ``pil_resize`` is compared bit for bit with Pillow itself (the library is installed;
pinned version of the reference: pillow 11.3.0, same algorithm) on random images over up- and down-scaling ratios,
both filters, sizes down to 1 pixel; ``smart_resize`` against its three defining properties, hand-computed cases, an
exhaustive scan for the rounding branch, and 400 size / limit combinations tabulated from the library's own
``smart_resize`` (transformers 5.15.0, tests/golden/processor_vectors.npz; tests/test_oracle_pixels.py).
"""

from __future__ import annotations

import math

import numpy as np

PRECISION_BITS = 32 - 8 - 2  # Resample.c: 8 bits of pixel, 2 bits of head-room
BILINEAR, BICUBIC = "bilinear", "bicubic"
_SUPPORT = {BILINEAR: 1.0, BICUBIC: 2.0}


def _filter(name: str, x: float) -> float:
    x = abs(x)
    if name == BILINEAR:
        return 1.0 - x if x < 1.0 else 0.0
    a = -0.5  # Resample.c bicubic_filter
    if x < 1.0:
        return ((a + 2.0) * x - (a + 3.0)) * x * x + 1
    if x < 2.0:
        return (((x - 5) * x + 8) * x - 4) * a
    return 0.0


def resample_coefficients(in_size: int, out_size: int, name: str):
    """Resample.c precompute_coeffs + normalize_coeffs_8bpc for the whole axis (box = the full image).
    Returns (bounds [out_size, 2] int32: first input index and tap count; kk [out_size, ksize] int32 fixed point)."""
    scale = in_size / out_size
    filterscale = scale if scale >= 1.0 else 1.0
    support = _SUPPORT[name] * filterscale
    ksize = int(math.ceil(support)) * 2 + 1
    bounds = np.zeros((out_size, 2), dtype=np.int32)
    kk = np.zeros((out_size, ksize), dtype=np.int32)
    ss = 1.0 / filterscale
    for xx in range(out_size):
        center = (xx + 0.5) * scale
        xmin = int(center - support + 0.5)
        if xmin < 0:
            xmin = 0
        xmax = int(center + support + 0.5)
        if xmax > in_size:
            xmax = in_size
        xmax -= xmin
        w = [_filter(name, (x + xmin - center + 0.5) * ss) for x in range(xmax)]
        ww = 0.0
        for v in w:
            ww += v
        if ww != 0.0:
            w = [v / ww for v in w]
        for x, v in enumerate(w):
            kk[xx, x] = int(-0.5 + v * (1 << PRECISION_BITS)) if v < 0 else int(0.5 + v * (1 << PRECISION_BITS))
        bounds[xx] = (xmin, xmax)
    return bounds, kk


def _pass(img: np.ndarray, out_size: int, name: str, axis: int) -> np.ndarray:
    """One resampling pass along ``axis`` of a uint8 [H, W, C] image (ImagingResampleHorizontal/Vertical_8bpc)."""
    bounds, kk = resample_coefficients(img.shape[axis], out_size, name)
    src = np.moveaxis(img, axis, 0).astype(np.int64)
    out = np.empty((out_size,) + src.shape[1:], dtype=np.uint8)
    for xx in range(out_size):
        xmin, n = int(bounds[xx, 0]), int(bounds[xx, 1])
        acc = np.full(src.shape[1:], 1 << (PRECISION_BITS - 1), dtype=np.int64)
        for x in range(n):
            acc += src[xmin + x] * int(kk[xx, x])
        out[xx] = np.clip(acc >> PRECISION_BITS, 0, 255).astype(np.uint8)  # clip8: arithmetic shift, then clamp
    return np.moveaxis(out, 0, axis)


def pil_resize(img: np.ndarray, out_h: int, out_w: int, name: str) -> np.ndarray:
    """``PIL.Image.fromarray(img).resize((out_w, out_h), resample)`` for a uint8 [H, W, 3] image: horizontal pass first,
    each pass skipped when the size along it does not change (ImagingResample)."""
    if img.dtype != np.uint8 or img.ndim != 3:
        raise ValueError("pil_resize: uint8 [H, W, C] image expected")
    if img.shape[1] != out_w:
        img = _pass(img, out_w, name, axis=1)
    if img.shape[0] != out_h:
        img = _pass(img, out_h, name, axis=0)
    return img


def smart_resize(height: int, width: int, factor: int = 28, min_pixels: int = 56 * 56, max_pixels: int = 14 * 14 * 4 * 1280):
    """Target (height, width) of the image processor's resize (image_processing_qwen2_vl.py smart_resize)."""
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
