"""Writes tests/golden/processor_vectors.npz from the image processor of the installed transformers.

Run once, in the build container (the library is importable there; it does not travel with the tests):

    python tests/golden/make_processor_vectors.py

What it records: ``transformers.models.qwen2_vl.image_processing_pil_qwen2_vl`` (transformers 5.15.0, PIL backend;
the reference pins transformers 4.57.0, which is absent, and reaches the same processor class family through
``processor.apply_chat_template``, python/data/preprocessing.py:134) is run on seeded uint8 images, and for each case
the file keeps the recipe of the input (a counter hashed with splitmix64, so that no random-number library has to
reproduce a stream), the target size, ``image_grid_thw``, the SHA-256 of the float32 ``pixel_values`` bytes and a
handful of sampled rows.  ``smart_resize`` itself is tabulated on a few hundred size / limit combinations.
Data only: no text of the library or of the reference is stored.
"""

from __future__ import annotations

import hashlib
from pathlib import Path

import numpy as np

OUT = Path(__file__).resolve().parent / "processor_vectors.npz"

# (name, height, width, min_pixels, max_pixels); None = the processor's defaults (3136, 1003520)
CASES = [
    ("no_resize_56x84", 56, 84, None, None),
    ("no_resize_224x224", 224, 224, None, None),
    ("round_to_28_300x500", 300, 500, None, None),
    ("downscale_2000x3000", 2000, 3000, None, None),
    ("min_pixels_clamp_30x40", 30, 40, None, None),
    ("upscale_thin_100x37", 100, 37, None, None),
    ("custom_limits_640x480", 640, 480, 56 * 56, 28 * 28 * 64),
    ("custom_limits_up_90x120", 90, 120, 28 * 28 * 100, 28 * 28 * 400),
]


def seeded_image(seed: int, height: int, width: int) -> np.ndarray:
    """[H, W, 3] uint8 from splitmix64 of a counter: identical on any numpy."""
    n = height * width * 3
    z = np.arange(n, dtype=np.uint64) + np.uint64((seed * 0x9E3779B97F4A7C15) % 2**64)
    with np.errstate(over="ignore"):
        z = (z + np.uint64(0x9E3779B97F4A7C15))
        z = (z ^ (z >> np.uint64(30))) * np.uint64(0xBF58476D1CE4E5B9)
        z = (z ^ (z >> np.uint64(27))) * np.uint64(0x94D049BB133111EB)
        z = z ^ (z >> np.uint64(31))
    return (z >> np.uint64(56)).astype(np.uint8).reshape(height, width, 3)


def main() -> None:
    import transformers
    from PIL import Image
    from transformers.models.qwen2_vl import image_processing_pil_qwen2_vl as lib

    out = {"transformers_version": np.array(transformers.__version__), "case_names": np.array([c[0] for c in CASES])}
    for i, (name, h, w, lo, hi) in enumerate(CASES):
        img = seeded_image(100 + i, h, w)
        kw = {}
        if lo is not None:
            kw["size"] = {"shortest_edge": lo, "longest_edge": hi}
        proc = lib.Qwen2VLImageProcessorPil(**kw)
        res = proc(images=[Image.fromarray(img)], return_tensors="np")
        pv = np.ascontiguousarray(res["pixel_values"], dtype=np.float32)
        grid = np.asarray(res["image_grid_thw"], dtype=np.int64)
        assert pv.dtype == np.float32 and pv.shape == (int(grid.prod()), 1176), (pv.dtype, pv.shape, grid)
        rows = np.unique(np.linspace(0, pv.shape[0] - 1, 6).astype(np.int64))
        out[f"{name}/recipe"] = np.array([100 + i, h, w, lo or 3136, hi or 1003520], dtype=np.int64)
        out[f"{name}/input_sha256"] = np.array(hashlib.sha256(img.tobytes()).hexdigest())
        out[f"{name}/grid_thw"] = grid
        out[f"{name}/pixel_values_sha256"] = np.array(hashlib.sha256(pv.tobytes()).hexdigest())
        out[f"{name}/sample_rows"] = rows
        out[f"{name}/sample_values"] = pv[rows]
        print(f"{name}: {h}x{w} -> grid {grid.tolist()}, {pv.shape[0]} rows")

    # smart_resize, tabulated: random sizes under the default limits and under random limits
    rng_sizes = seeded_image(7, 40, 40).astype(np.int64).reshape(-1)
    table = []
    for j in range(400):
        a, b, c, d, e = (int(x) for x in rng_sizes[5 * j:5 * j + 5])
        h = 20 + a * 11 + b % 11
        w = 20 + c * 11 + d % 11
        if j % 2:
            lo, hi = 3136, 1003520
        else:
            lo = 28 * 28 * (1 + e % 64)
            hi = lo * (1 + (a + c) % 40)
        if max(h, w) / min(h, w) > 200:
            continue
        table.append([h, w, lo, hi, *lib.smart_resize(h, w, 28, lo, hi)])
    out["smart_resize_table"] = np.asarray(table, dtype=np.int64)
    np.savez_compressed(OUT, **out)
    print(f"wrote {OUT} ({OUT.stat().st_size} bytes), smart_resize cases: {len(table)}")


if __name__ == "__main__":
    main()
