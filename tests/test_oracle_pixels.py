"""Pins oracle/pixels_oracle.py (decoded frames -> pixel_values rows) without the image-processor library, which is
not importable here: row order against the position ids the model computes for each row, column order against
Conv3d (the patch embedding the model applies), the arithmetic against its closed form, and the frame fill-up."""

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
