"""CPU restatement of the input side: decoded frames -> ``pixel_values`` rows.

TEST INFRASTRUCTURE ONLY (see ``oracle/__init__.py``).

The reference does not hold this code: ``python/data/preprocessing.py:134`` calls
``processor.apply_chat_template(..., tokenize=True)``, which runs the image processor of
``transformers`` (pinned ``transformers==4.57.0`` in the reference's requirements.txt;
``models/qwen2_vl/image_processing_qwen2_vl.py``, ``Qwen2VLImageProcessor._preprocess``),
and ``python/data/collator.py:134-156`` concatenates the per-sample results along dim 0.
Version 4.57.0 is not installed; the installed transformers 5.15.0 holds the same processor with a PIL
backend (``models/qwen2_vl/image_processing_pil_qwen2_vl.py``, ``Qwen2VLImageProcessorPil``), and the
restatement below is held to it bit for bit.  The algorithm, for frames that are already resized
(height and width multiples of patch * merge = 28):

  1. rescale: ``image.astype(float64) * (1 / 255)`` cast to float32   (image_transforms.rescale)
  2. normalise: ``(image - mean) / std`` in float32, mean / std = OPENAI_CLIP  (image_transforms.normalize)
  3. frames -> channels first; a frame count that is not a multiple of ``temporal_patch_size``
     is filled up by repeating the last frame (a still image is one frame, used twice)
  4. reshape to (grid_t, tps, C, grid_h/m, m, ps, grid_w/m, m, ps), transpose to
     (grid_t, grid_h/m, grid_w/m, m, m, C, tps, ps, ps), flatten to
     [grid_t * grid_h * grid_w, C * tps * ps * ps] = [rows, 1176]

What pins each part besides its own formula (tests/test_oracle_pixels.py):

===================  ==============================================================
row order            row r of an image is the patch at (h, w) = ``rot_pos_ids`` row r,
                     the position ids the reference's model computes for that row
                     (modeling_qwen2_5_vl.py rot_pos_emb, restated in vit_oracle and
                     pinned there): the merge-block order both sides must share
column order         ``rows @ W.view(1280, 1176).T`` equals ``torch.nn.functional.conv3d``
                     of the normalised [C, T, H, W] volume with kernel = stride =
                     (2, 14, 14): the patch embedding the reference applies to it
                     (Qwen2_5_VisionPatchEmbed: Conv3d on rows viewed as
                     [-1, 3, 2, 14, 14])
rescale / normalise  closed form in float64, agreement to 1 float32 ulp
the whole chain      ``smart_resize`` -> bicubic resize (oracle/resize_oracle.py) -> these rows
                     equal ``Qwen2VLImageProcessorPil()(images=...)`` of transformers 5.15.0
                     bit for bit (SHA-256 of the float32 ``pixel_values`` and sampled rows)
                     on eight seeded images: no resize, rounding to multiples of 28,
                     a 2000 x 3000 down-scale, the min-pixels clamp, a thin up-scale,
                     custom pixel limits; vectors in tests/golden/processor_vectors.npz,
                     written by tests/golden/make_processor_vectors.py.  Against 4.57.0
                     itself (the reference's pin): not checked, that version is absent
frame fill-up        still image: both temporal halves of a row equal; odd videos:
                     last row group uses the last frame twice
===================  ==============================================================
"""

from __future__ import annotations

from typing import List, Sequence, Tuple

import numpy as np

OPENAI_CLIP_MEAN = (0.48145466, 0.4578275, 0.40821073)
OPENAI_CLIP_STD = (0.26862954, 0.26130258, 0.27577711)
PATCH, TEMPORAL_PATCH, MERGE = 14, 2, 2


def grid_of(frames: int, height: int, width: int, patch: int = PATCH, tps: int = TEMPORAL_PATCH) -> Tuple[int, int, int]:
    """(grid_t, grid_h, grid_w) of already resized frames."""
    return (frames + tps - 1) // tps, height // patch, width // patch


def normalise(frames_u8: np.ndarray, mean: Sequence[float] = OPENAI_CLIP_MEAN, std: Sequence[float] = OPENAI_CLIP_STD,
              scale: float = 1.0 / 255.0) -> np.ndarray:
    """[F, H, W, 3] uint8 -> float32, steps 1 and 2 with the library's dtypes."""
    x = (frames_u8.astype(np.float64) * scale).astype(np.float32)
    return (x - np.asarray(mean, dtype=np.float32)) / np.asarray(std, dtype=np.float32)


def patchify(frames_u8: np.ndarray, mean: Sequence[float] = OPENAI_CLIP_MEAN, std: Sequence[float] = OPENAI_CLIP_STD,
             patch: int = PATCH, tps: int = TEMPORAL_PATCH, merge: int = MERGE,
             scale: float = 1.0 / 255.0) -> Tuple[np.ndarray, Tuple[int, int, int]]:
    """One image or video, [F, H, W, 3] uint8 -> ([grid_t*grid_h*grid_w, 3*tps*patch*patch] float32, grid)."""
    assert frames_u8.dtype == np.uint8 and frames_u8.ndim == 4 and frames_u8.shape[3] == 3
    f, h, w, _ = frames_u8.shape
    assert h % (patch * merge) == 0 and w % (patch * merge) == 0, "frames must be resized to multiples of patch * merge"
    x = normalise(frames_u8, mean, std, scale).transpose(0, 3, 1, 2)  # [F, C, H, W]
    if f % tps != 0:
        x = np.concatenate([x, np.repeat(x[-1][None], tps - f % tps, axis=0)], axis=0)
    gt, gh, gw = x.shape[0] // tps, h // patch, w // patch
    x = x.reshape(gt, tps, 3, gh // merge, merge, patch, gw // merge, merge, patch)
    x = x.transpose(0, 3, 6, 4, 7, 2, 1, 5, 8)
    return np.ascontiguousarray(x.reshape(gt * gh * gw, 3 * tps * patch * patch)), (gt, gh, gw)


def patchify_batch(images: List[np.ndarray], **kw) -> Tuple[np.ndarray, np.ndarray]:
    """Several images / videos -> (rows concatenated along dim 0 as the collator does, grid_thw [n, 3] int64)."""
    rows, grids = zip(*(patchify(im, **kw) for im in images))
    return np.concatenate(rows, axis=0), np.asarray(grids, dtype=np.int64)
