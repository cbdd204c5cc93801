"""Pins oracle/pixels_oracle.py (decoded frames -> pixel_values rows): row order against the position ids the model
computes for each row, column order against Conv3d (the patch embedding the model applies), the arithmetic against its
closed form, the frame fill-up, and the whole chain (target size, bicubic resize, rescale, normalise, patch rows)
against vectors written from the image-processor library itself (second half of this file)."""

import numpy as np
import pytest
import torch

from oracle import pixels_oracle as po
from oracle import vit_oracle as vo


def _frames(seed, f, h, w):
    return np.random.default_rng(seed).integers(0, 256, size=(f, h, w, 3), dtype=np.uint8)


def _denorm(v, c):
    return v * np.float32(po.OPENAI_CLIP_STD[c]) + np.float32(po.OPENAI_CLIP_MEAN[c])


@pytest.mark.parametrize("h,w", [(56, 84), (112, 28), (28, 28), (140, 196)])
def test_row_order_is_the_models_position_id_order(h, w):
    """Red encodes the patch row, green the patch column: row r must show rot_pos_ids[r]."""
    img = np.zeros((1, h, w, 3), dtype=np.uint8)
    img[0, :, :, 0] = (np.arange(h) // po.PATCH)[:, None]
    img[0, :, :, 1] = (np.arange(w) // po.PATCH)[None, :]
    rows, grid = po.patchify(img)
    assert grid == (1, h // 14, w // 14) and rows.shape == (grid[1] * grid[2], 1176)
    ids = vo.rot_pos_ids([grid], po.MERGE).numpy()
    r = rows.reshape(-1, 3, 2, 14, 14)
    got_h = np.rint(_denorm(r[:, 0], 0) * 255.0)
    got_w = np.rint(_denorm(r[:, 1], 1) * 255.0)
    assert (got_h == ids[:, 0][:, None, None, None]).all()  # every element of the patch, both temporal halves
    assert (got_w == ids[:, 1][:, None, None, None]).all()


@pytest.mark.parametrize("f,h,w", [(1, 56, 84), (2, 84, 56), (3, 28, 56), (4, 56, 56)])
def test_column_order_is_conv3d_patch_embedding(f, h, w):
    frames = _frames(1, f, h, w)
    rows, (gt, gh, gw) = po.patchify(frames)
    weight = torch.randn(8, 3, 2, 14, 14, generator=torch.Generator().manual_seed(2))
    x = torch.from_numpy(po.normalise(frames)).permute(3, 0, 1, 2)  # [C, F, H, W]
    if f % 2:
        x = torch.cat([x, x[:, -1:]], dim=1)
    ref = torch.nn.functional.conv3d(x[None], weight, stride=(2, 14, 14))[0]  # [8, gt, gh, gw]
    got = torch.from_numpy(rows) @ weight.view(8, -1).T  # [rows, 8], rows in (t, merge-block) order
    ids = vo.rot_pos_ids([(gt, gh, gw)], po.MERGE)
    t_of_row = torch.arange(gt).repeat_interleave(gh * gw)
    want = ref[:, t_of_row, ids[:, 0], ids[:, 1]].T
    assert vo.max_rel_err(got, want) <= 1e-5


def test_arithmetic_closed_form_and_dtype():
    frames = np.arange(256, dtype=np.uint8).reshape(1, 16, 16, 1).repeat(3, axis=3)
    got = po.normalise(frames)
    assert got.dtype == np.float32
    want = (frames.astype(np.float64) / 255.0 - np.asarray(po.OPENAI_CLIP_MEAN)) / np.asarray(po.OPENAI_CLIP_STD)
    assert np.abs(got - want).max() <= 3e-7  # two float32 roundings of values below 2.7, divided by std >= 0.26
    assert got[0, 0, 0, 0] == np.float32(-0.48145466) / np.float32(0.26862954)  # x = 0: -mean / std in float32
    # known answers of the published constants: x = 255 -> (1 - mean) / std
    assert np.allclose(got[0, 15, 15], [1.9303361, 2.0748837, 2.1458969], rtol=0, atol=2e-6)


def test_frame_fill_up():
    still, _ = po.patchify(_frames(3, 1, 28, 56))
    s = still.reshape(-1, 3, 2, 196)
    assert np.array_equal(s[:, :, 0], s[:, :, 1])  # a still image is used for both temporal halves
    frames = _frames(4, 3, 28, 28)
    rows, grid = po.patchify(frames)
    assert grid == (2, 2, 2) and rows.shape == (8, 1176)
    r = rows.reshape(2, 4, 3, 2, 196)
    assert np.array_equal(r[1, :, :, 0], r[1, :, :, 1])  # frames 2, 2
    assert not np.array_equal(r[0, :, :, 0], r[0, :, :, 1])  # frames 0, 1
    pair, _ = po.patchify(frames[:2])
    assert np.array_equal(rows[:4], pair)


def test_batch_concatenates_like_the_collator_and_rejects_unresized_frames():
    a, b = _frames(5, 1, 56, 28), _frames(6, 2, 28, 84)
    rows, grids = po.patchify_batch([a, b])
    assert grids.tolist() == [[1, 4, 2], [1, 2, 6]] and rows.shape == (20, 1176)
    assert np.array_equal(rows[:8], po.patchify(a)[0]) and np.array_equal(rows[8:], po.patchify(b)[0])
    with pytest.raises(AssertionError):
        po.patchify(_frames(7, 1, 30, 28))


def test_host_mirror_grid_and_guards_without_a_gpu():
    """mi355_vit.pixels: the grid it reports equals the oracle's, and what it cannot do is refused before any launch."""
    from mi355_vit import pixels

    frames = [torch.zeros(f, h, w, 3, dtype=torch.uint8) for f, h, w in [(1, 56, 84), (3, 28, 112), (4, 140, 28)]]
    assert pixels.grid_thw_of(frames).tolist() == [list(po.grid_of(*f.shape[:3])) for f in frames]
    assert pixels.OPENAI_CLIP_MEAN == po.OPENAI_CLIP_MEAN and pixels.OPENAI_CLIP_STD == po.OPENAI_CLIP_STD
    for bad in (torch.zeros(1, 30, 28, 3, dtype=torch.uint8), torch.zeros(1, 28, 28, 4, dtype=torch.uint8),
                torch.zeros(28, 28, 3, dtype=torch.uint8), torch.zeros(1, 28, 28, 3), torch.zeros(0, 28, 28, 3, dtype=torch.uint8)):
        with pytest.raises(ValueError):
            pixels.grid_thw_of([bad])
    with pytest.raises(RuntimeError, match="no CPU path"):
        pixels.patchify(frames[:1])


# ---- the oracle against the image processor library itself ------------------------------------------------------
# tests/golden/processor_vectors.npz is written by tests/golden/make_processor_vectors.py from
# transformers.models.qwen2_vl.image_processing_pil_qwen2_vl (transformers 5.15.0; the reference's pin, 4.57.0, is
# not installed): target sizes, grids and the float32 pixel_values (as SHA-256 plus sampled rows) of seeded images.

def _processor_vectors():
    import importlib.util
    from pathlib import Path

    golden = Path(__file__).resolve().parent / "golden"
    spec = importlib.util.spec_from_file_location("make_processor_vectors", golden / "make_processor_vectors.py")
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod, np.load(golden / "processor_vectors.npz")


def _case_names():
    return [c[0] for c in _processor_vectors()[0].CASES]


@pytest.mark.parametrize("name", _case_names())
def test_resize_and_patch_rows_equal_the_library_bit_for_bit(name):
    import hashlib

    from oracle import resize_oracle as ro

    mod, vec = _processor_vectors()
    seed, h, w, lo, hi = (int(x) for x in vec[f"{name}/recipe"])
    img = mod.seeded_image(seed, h, w)
    assert hashlib.sha256(img.tobytes()).hexdigest() == str(vec[f"{name}/input_sha256"])
    th, tw = ro.smart_resize(h, w, 28, lo, hi)
    grid = vec[f"{name}/grid_thw"]
    assert grid.tolist() == [[1, th // 14, tw // 14]]
    resized = img if (th, tw) == (h, w) else ro.pil_resize(img, th, tw, ro.BICUBIC)
    rows, g = po.patchify(resized[None])
    assert list(g) == grid[0].tolist() and rows.dtype == np.float32
    sample = vec[f"{name}/sample_rows"]
    assert np.array_equal(rows[sample], vec[f"{name}/sample_values"])
    assert hashlib.sha256(np.ascontiguousarray(rows).tobytes()).hexdigest() == str(vec[f"{name}/pixel_values_sha256"])


def test_smart_resize_equals_the_library_on_its_table():
    from oracle import resize_oracle as ro

    table = _processor_vectors()[1]["smart_resize_table"]
    assert len(table) >= 300
    for h, w, lo, hi, th, tw in table.tolist():
        assert ro.smart_resize(h, w, 28, lo, hi) == (th, tw), (h, w, lo, hi)


def test_processor_vectors_discriminate():
    """A plausible mistake in the oracle must fail the vectors: truncating instead of rounding the rescale, or the
    bilinear filter in place of the bicubic one."""
    from oracle import resize_oracle as ro

    mod, vec = _processor_vectors()
    name = "round_to_28_300x500"
    seed, h, w, lo, hi = (int(x) for x in vec[f"{name}/recipe"])
    img = mod.seeded_image(seed, h, w)
    th, tw = ro.smart_resize(h, w, 28, lo, hi)
    sample = vec[f"{name}/sample_rows"]
    wrong_filter, _ = po.patchify(ro.pil_resize(img, th, tw, ro.BILINEAR)[None])
    assert not np.array_equal(wrong_filter[sample], vec[f"{name}/sample_values"])
    resized = ro.pil_resize(img, th, tw, ro.BICUBIC)

    def rescale_in_float32(frames_u8, mean=po.OPENAI_CLIP_MEAN, std=po.OPENAI_CLIP_STD, scale=1.0 / 255.0):
        x = frames_u8.astype(np.float32) * np.float32(scale)  # the library multiplies in float64 and rounds once
        return (x - np.asarray(mean, dtype=np.float32)) / np.asarray(std, dtype=np.float32)

    right = po.normalise
    try:
        po.normalise = rescale_in_float32
        wrong_rescale, _ = po.patchify(resized[None])
    finally:
        po.normalise = right
    assert not np.array_equal(wrong_rescale[sample], vec[f"{name}/sample_values"])
    good, _ = po.patchify(resized[None])
    assert np.array_equal(good[sample], vec[f"{name}/sample_values"])
