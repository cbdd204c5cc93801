"""Parity of the input-side kernel (decoded frames -> pixel_values rows, through the C ABI) against the CPU oracle.

float32 output is compared bit for bit (the oracle restates the image processor's arithmetic with its dtypes);
bfloat16 output bit for bit against the oracle's float32 result rounded once, the cast the tower applies."""

import numpy as np
import pytest
import torch

from oracle import pixels_oracle as po

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _announce(msg):
    print(f"[case] {msg}", flush=True)


def _batch(seed, shapes):
    rng = np.random.default_rng(seed)
    return [rng.integers(0, 256, size=(f, h, w, 3), dtype=np.uint8) for f, h, w in shapes]


def _run(images, **kw):
    from mi355_vit.pixels import patchify

    out, grid = patchify([torch.from_numpy(im).to(DEV) for im in images], **kw)
    torch.cuda.synchronize()
    return out.cpu(), grid


RAGGED = [(1, 56, 84), (1, 28, 28), (2, 84, 56), (3, 28, 112), (1, 364, 252), (5, 56, 56), (1, 112, 28)]


@pytest.mark.parametrize("seed", [0, 1])
def test_patchify_bit_exact_against_oracle_ragged_images_and_videos(seed):
    _announce(f"patchify fp32 ragged seed={seed}")
    images = _batch(seed, RAGGED)
    got, grid = _run(images)
    ref, ref_grid = po.patchify_batch(images)
    assert grid.dtype == torch.int64 and not grid.is_cuda and grid.tolist() == ref_grid.tolist()
    assert got.dtype == torch.float32 and tuple(got.shape) == ref.shape
    assert np.array_equal(got.numpy().view(np.uint32), ref.view(np.uint32))


def test_patchify_bf16_is_the_rounded_fp32_result():
    _announce("patchify bf16")
    images = _batch(2, RAGGED[:5])
    got, _ = _run(images, dtype=torch.bfloat16)
    ref = torch.from_numpy(po.patchify_batch(images)[0]).to(torch.bfloat16)
    assert got.dtype == torch.bfloat16 and torch.equal(got, ref)


def test_patchify_every_byte_value_other_constants_and_out_argument():
    _announce("patchify all byte values, custom constants")
    ramp = np.arange(28 * 28 * 3, dtype=np.int64).reshape(1, 28, 28, 3) % 256
    images = [ramp.astype(np.uint8), _batch(3, [(2, 28, 56)])[0]]
    mean, std, scale = (0.5, 0.25, 0.125), (0.5, 0.3, 0.7), 1.0 / 127.5
    from mi355_vit.pixels import patchify

    out = torch.full((4 + 8, 1176), float("nan"), device=DEV)
    got, _ = patchify([torch.from_numpy(im).to(DEV) for im in images], image_mean=mean, image_std=std, rescale_factor=scale, out=out)
    assert got.data_ptr() == out.data_ptr()
    ref = np.concatenate([po.patchify(im, mean=mean, std=std, scale=scale)[0] for im in images])
    assert np.array_equal(got.cpu().numpy().view(np.uint32), ref.view(np.uint32))


def test_patchify_frames_at_an_odd_address():
    """Frame buffers that are views one byte into an allocation: no dword alignment, byte path of the staging."""
    from mi355_vit.pixels import patchify

    _announce("patchify misaligned frames")
    images = _batch(6, [(1, 56, 28), (3, 28, 84)])
    views = []
    for im in images:
        buf = torch.zeros(im.size + 1, dtype=torch.uint8, device=DEV)
        buf[1:].copy_(torch.from_numpy(im).reshape(-1))
        views.append(buf[1:].view(im.shape))
        assert views[-1].data_ptr() % 4 == 1
    got, _ = patchify(views)
    ref, _ = po.patchify_batch(images)
    assert np.array_equal(got.cpu().numpy().view(np.uint32), ref.view(np.uint32))


def test_patchify_full_benchmark_batch():
    """The 8 ragged images of the benchmark workload (25,524 rows): bit-exact, and a still image fills both halves."""
    _announce("patchify cfg2 batch")
    grids = [[1, 76, 60], [1, 86, 54], [1, 82, 34], [1, 42, 78], [1, 54, 32], [1, 72, 56], [1, 40, 42], [1, 64, 44]]
    images = _batch(4, [(1, 14 * h, 14 * w) for _, h, w in grids])
    got, grid = _run(images)
    assert grid.tolist() == grids and got.shape == (25524, 1176)
    ref, _ = po.patchify_batch(images)
    assert np.array_equal(got.numpy().view(np.uint32), ref.view(np.uint32))
    halves = got.view(-1, 3, 2, 196)
    assert torch.equal(halves[:, :, 0], halves[:, :, 1])


def test_patchify_feeds_the_tower():
    """pixel_values made on the GPU give the same tower output as the oracle's rows (same bits in, same bits out)."""
    from mi355_vit.config import Qwen2_5_VLVisionConfig
    from mi355_vit.modeling import Qwen2_5_VisionTransformerPretrainedModel
    from mi355_vit.pixels import patchify

    _announce("patchify -> tower")
    images = _batch(5, [(1, 56, 84), (2, 56, 56)])
    cfg = Qwen2_5_VLVisionConfig(depth=2, hidden_size=256, intermediate_size=300, num_heads=8, out_hidden_size=256,
                                 window_size=56, fullatt_block_indexes=[1])
    torch.manual_seed(0)
    tower = Qwen2_5_VisionTransformerPretrainedModel(cfg).to(torch.bfloat16).to(DEV)
    pv, grid = patchify([torch.from_numpy(im).to(DEV) for im in images], dtype=torch.bfloat16)
    ref_pv = torch.from_numpy(po.patchify_batch(images)[0]).to(DEV)  # float32: the tower casts it as its first step
    with torch.no_grad():
        a = tower(pv, grid)
        b = tower(ref_pv, grid)
    assert torch.equal(a, b)


def test_trainer_takes_frames_batches():
    """VisionTrainer.forward_step with a batch of uint8 frames equals the same step fed the oracle's pixel_values."""
    from mi355_vit.trainer import VisionTrainer

    _announce("trainer with frames batches")
    cfg = dict(seed=0, parallelism="none", dtype="bfloat16", autocast=False, learning_rate=1e-3, weight_decay=0.0,
               warmup_ratio=0.0, warmup_steps=0, lr_scheduler_type="constant", num_iterations=2, max_grad_norm=1.0,
               activation_checkpointing=False, model_name=None,
               vision_config=dict(depth=2, hidden_size=256, intermediate_size=300, num_heads=8, out_hidden_size=256,
                                  window_size=56, fullatt_block_indexes=[1]))
    images = _batch(7, [(1, 56, 84), (3, 28, 56)])
    rows, grid = po.patchify_batch(images)
    outs = []
    for batch in ({"frames": [torch.from_numpy(im) for im in images], "sample_index": torch.tensor([0])},
                  {"pixel_values": torch.from_numpy(rows), "image_grid_thw": torch.from_numpy(grid), "sample_index": torch.tensor([0])}):
        tr = VisionTrainer(cfg, rank=0)
        tr.build_model()
        tr.set_data_iterator([batch])
        tr.initialize_trainer()
        outs.append(tr.forward_step(0)["vision_embeddings"].detach().clone())
    # the frames path contracts the patch embedding in another order (along memory): same values up to bf16 rounding
    err = (outs[0].float() - outs[1].float()).abs().max() / outs[1].float().abs().max()
    assert err < 1e-2, err
    # with the fusion switched off the two paths run the same kernels on the same bits
    from mi355_vit.modeling import Qwen2_5_VisionPatchEmbed

    Qwen2_5_VisionPatchEmbed.fuse_frames = False
    try:
        tr = VisionTrainer(cfg, rank=0)
        tr.build_model()
        tr.set_data_iterator([{"frames": [torch.from_numpy(im) for im in images], "sample_index": torch.tensor([0])}])
        tr.initialize_trainer()
        assert torch.equal(tr.forward_step(0)["vision_embeddings"], outs[1])
    finally:
        Qwen2_5_VisionPatchEmbed.fuse_frames = True


def test_patchify_rejects_what_it_cannot_do():
    from mi355_vit.pixels import patchify

    ok = torch.zeros(1, 28, 28, 3, dtype=torch.uint8, device=DEV)
    with pytest.raises(RuntimeError, match="no CPU path"):
        patchify([ok.cpu()])
    with pytest.raises(ValueError, match="multiples of 28"):
        patchify([torch.zeros(1, 30, 28, 3, dtype=torch.uint8, device=DEV)])
    with pytest.raises(ValueError, match="uint8"):
        patchify([ok.float()])
    with pytest.raises(TypeError):
        patchify([ok], dtype=torch.float16)
    with pytest.raises(ValueError, match="no images"):
        patchify([])
    with pytest.raises(RuntimeError, match="contiguous"):
        patchify([torch.zeros(1, 28, 56, 3, dtype=torch.uint8, device=DEV)[:, :, ::2]])


# ------------------------------------------------------------------------------- patch embedding from frames


def _bf16_rows_f64(images):
    """pixel_values of the oracle, rounded to bfloat16 (what the tower multiplies), as float64."""
    return torch.from_numpy(po.patchify_batch(images)[0]).to(torch.bfloat16).to(torch.float64)


def test_pack_patch_embed_weight_is_the_documented_permutation():
    from mi355_vit.pixels import pack_patch_embed_weight

    _announce("pack patch-embed weight")
    torch.manual_seed(0)
    for dtype in (torch.bfloat16, torch.float32):
        w = torch.randn(40, 3, 2, 14, 14, device=DEV).to(dtype)
        got = pack_patch_embed_weight(w).cpu()
        ref = torch.zeros(40, 28, 48, dtype=torch.bfloat16)
        # [n, channel, frame, y, x] -> [n, frame, y, x, channel] -> lines of 42 values
        ref[:, :, :42] = w.cpu().to(torch.bfloat16).permute(0, 2, 3, 4, 1).reshape(40, 28, 42)
        assert got.shape == (40, 1344) and torch.equal(got, ref.reshape(40, 1344))


@pytest.mark.parametrize("n_out,out_dtype", [(256, torch.float32), (200, torch.float32), (1280, torch.bfloat16)])
def test_patch_embed_frames_equals_bf16_rows_times_weight(n_out, out_dtype):
    """Ragged images and videos (odd frame counts, 616 rows = two full row tiles and a partial one): the fused kernel
    equals oracle rows rounded to bf16 times the weight, evaluated in float64, to fp32-accumulation accuracy; one
    operand element that differed by a bf16 ulp would show as ~1e-4 of the output scale."""
    from mi355_vit.pixels import pack_patch_embed_weight, patch_embed_frames

    _announce(f"patch_embed_frames ragged n_out={n_out} {out_dtype}")
    images = _batch(11, RAGGED)
    torch.manual_seed(1)
    w = (torch.randn(n_out, 1176) * 0.05).to(torch.bfloat16)
    got, grid = patch_embed_frames([torch.from_numpy(im).to(DEV) for im in images], pack_patch_embed_weight(w.to(DEV)), dtype=out_dtype)
    torch.cuda.synchronize()
    ref = _bf16_rows_f64(images) @ w.to(torch.float64).T
    assert grid.tolist() == po.patchify_batch(images)[1].tolist() and tuple(got.shape) == tuple(ref.shape)
    if out_dtype == torch.float32:
        err = (got.cpu().double() - ref).abs().max() / ref.abs().max()
        assert err < 2e-5, err
    else:
        assert got.dtype == torch.bfloat16
        # at most one bf16 ulp from the rounded exact result (fp32 accumulation can tip a value that lies at a rounding boundary)
        r = ref.to(torch.bfloat16).float()
        ulp = torch.maximum(r.abs(), torch.tensor(1e-3)) * 2.0 ** -7
        assert ((got.cpu().float() - r).abs() <= ulp).all()
        assert (got.cpu().float() != r).float().mean() < 0.02


def test_patch_embed_frames_full_benchmark_batch_against_the_two_kernel_path():
    """cfg2's 8 ragged images (25,524 rows) at the tower's width: fused kernel against patchify + GEMM on the GPU and,
    for sampled rows, against float64."""
    from mi355_vit import ops
    from mi355_vit.pixels import pack_patch_embed_weight, patch_embed_frames, patchify

    _announce("patch_embed_frames cfg2 batch")
    grids = [[1, 76, 60], [1, 86, 54], [1, 82, 34], [1, 42, 78], [1, 54, 32], [1, 72, 56], [1, 40, 42], [1, 64, 44]]
    images = _batch(4, [(1, 14 * h, 14 * w) for _, h, w in grids])
    frames = [torch.from_numpy(im).to(DEV) for im in images]
    torch.manual_seed(2)
    w = (torch.randn(1280, 1176, device=DEV) * 0.03).to(torch.bfloat16)
    got, grid = patch_embed_frames(frames, pack_patch_embed_weight(w), dtype=torch.float32)
    rows, _ = patchify(frames, dtype=torch.bfloat16)
    two = torch.empty(rows.shape[0], 1280, dtype=torch.float32, device=DEV)
    ops.gemm(rows, w, two)
    torch.cuda.synchronize()
    assert grid.tolist() == grids and got.shape == (25524, 1280)
    scale = two.abs().max()
    assert (got - two).abs().max() / scale < 2e-5
    pick = torch.tensor([0, 1, 255, 256, 4559, 4560, 12000, 25523])
    ref = rows[pick.to(DEV)].cpu().double() @ w.cpu().double().T
    assert (got[pick.to(DEV)].cpu().double() - ref).abs().max() / ref.abs().max() < 2e-5


def _affine_fold_is_exact(mean, std, scale):
    """Whether byte * a + c (one fused multiply-add, float32) rounds to the same bfloat16 as the processor's
    (float32(byte * scale) - mean) / std for every byte and channel: the library's own acceptance test, in numpy."""
    def bf16_bits(x):
        u = np.asarray(x, np.float32).view(np.uint32).astype(np.uint64)
        return ((u + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint32)

    b = np.arange(256)
    for m, s in zip(mean, std):
        m, s = np.float32(m), np.float32(s)
        table = (((b.astype(np.float64) * scale).astype(np.float32) - m) / s).astype(np.float32)
        a = np.float32(np.float64(scale) / np.float64(s))
        c = np.float32(-np.float64(m) / np.float64(s))
        affine = (b.astype(np.float64) * np.float64(a) + np.float64(c)).astype(np.float32)  # exact product and sum, one rounding
        if not np.array_equal(bf16_bits(table), bf16_bits(affine)):
            return False
    return True


def test_patch_embed_frames_refuses_constants_it_cannot_fold_and_the_module_falls_back():
    from mi355_vit import _lib
    from mi355_vit.pixels import OPENAI_CLIP_MEAN, OPENAI_CLIP_STD, pack_patch_embed_weight, patch_embed_frames

    _announce("patch_embed_frames constants check")
    assert _affine_fold_is_exact(OPENAI_CLIP_MEAN, OPENAI_CLIP_STD, 1.0 / 255.0)
    rng = np.random.default_rng(5)
    bad = None
    for _ in range(2000):
        mean, std = rng.uniform(0.2, 0.7, 3), rng.uniform(0.15, 0.4, 3)
        if not _affine_fold_is_exact(mean, std, 1.0 / 255.0):
            bad = (tuple(float(np.float32(x)) for x in mean), tuple(float(np.float32(x)) for x in std))
            break
    assert bad is not None
    frames = [torch.from_numpy(im).to(DEV) for im in _batch(8, [(1, 28, 56)])]
    pw = pack_patch_embed_weight(torch.randn(64, 1176, device=DEV).to(torch.bfloat16))
    with pytest.raises(_lib.Unsupported, match="does not round"):
        patch_embed_frames(frames, pw, image_mean=bad[0], image_std=bad[1])
    with pytest.raises(RuntimeError, match="4-byte aligned"):
        buf = torch.zeros(28 * 56 * 3 + 1, dtype=torch.uint8, device=DEV)
        patch_embed_frames([buf[1:].view(1, 28, 56, 3)], pw)
    with pytest.raises(ValueError, match="packed_weight"):
        patch_embed_frames(frames, pw[:, :1176].contiguous())


def test_tower_takes_frames_and_trains_the_patch_embedding():
    """model(frames=...) equals model(pixel_values from patchify) up to bf16 rounding, and every gradient, the patch
    embedding's included, matches; frames at an odd address take the two-kernel path and give the same bits as it."""
    from mi355_vit.config import Qwen2_5_VLVisionConfig
    from mi355_vit.modeling import Qwen2_5_VisionTransformerPretrainedModel
    from mi355_vit.pixels import patchify

    _announce("tower from frames")
    images = _batch(9, [(1, 56, 84), (3, 56, 56), (1, 28, 28)])
    frames = [torch.from_numpy(im).to(DEV) for im in images]
    cfg = Qwen2_5_VLVisionConfig(depth=2, hidden_size=256, intermediate_size=300, num_heads=8, out_hidden_size=256,
                                 window_size=56, fullatt_block_indexes=[1])
    torch.manual_seed(0)
    tower = Qwen2_5_VisionTransformerPretrainedModel(cfg).to(torch.bfloat16).to(DEV).train()
    pv, grid = patchify(frames, dtype=torch.bfloat16)
    gout = torch.randn(pv.shape[0] // 4, 256, device=DEV).to(torch.bfloat16)

    def run(**kw):
        tower.zero_grad(set_to_none=True)
        out = tower(**kw)
        out.backward(gout)
        return out.detach().float(), {n: p.grad.detach().float().clone() for n, p in tower.named_parameters()}

    out_f, g_f = run(frames=frames)
    out_r, g_r = run(hidden_states=pv, grid_thw=grid)
    assert (out_f - out_r).abs().max() / out_r.abs().max() < 1e-2
    for n in g_r:
        assert (g_f[n] - g_r[n]).abs().max() / g_r[n].abs().max().clamp_min(1e-20) < 2e-2, n
    assert g_f["patch_embed.proj.weight"].abs().max() > 0
    odd = []
    for im in images:
        buf = torch.zeros(im.size + 1, dtype=torch.uint8, device=DEV)
        buf[1:].copy_(torch.from_numpy(im).reshape(-1))
        odd.append(buf[1:].view(im.shape))
    out_o, g_o = run(frames=odd)
    assert torch.equal(out_o, out_r) and all(torch.equal(g_o[n], g_r[n]) for n in g_r)
    with pytest.raises(ValueError, match="either"):
        tower(hidden_states=pv, grid_thw=grid, frames=frames)
    with pytest.raises(ValueError, match="does not describe"):
        tower(frames=frames, grid_thw=torch.tensor([[1, 4, 6]]))


# ------------------------------------------------------------------------------------------------ resize


def _resize_gpu(img, oh, ow, name):
    from mi355_vit.pixels import resize_frames

    out = resize_frames(torch.from_numpy(img).to(DEV), oh, ow, name)
    torch.cuda.synchronize()
    return out.cpu().numpy()


@pytest.mark.parametrize("name", ["bilinear", "bicubic"])
def test_resize_bit_exact_against_oracle_and_pillow(name):
    """Up- and down-scaling, one pass skipped, videos (several frames), odd widths (the byte-wise path of the vertical
    pass), against the oracle and, where Pillow is installed, against PIL.Image.resize itself."""
    from oracle import resize_oracle as ro

    rng = np.random.default_rng(11)
    cases = [(1, 37, 53, 28, 56), (1, 100, 80, 56, 56), (2, 28, 28, 112, 84), (1, 5, 7, 28, 28), (3, 64, 64, 64, 32), (1, 64, 60, 28, 60),
             (1, 211, 157, 140, 196), (1, 33, 1, 28, 28), (1, 90, 61, 45, 33), (1, 300, 200, 299, 201),
             (1, 40, 400, 28, 56),    # windows of 17 / 31 taps: beyond what the column kernel keeps in registers
             (1, 70, 900, 28, 700)]   # three column blocks of 256 output pixels, 70 rows = three row strips
    try:
        from PIL import Image
        filt = {"bilinear": Image.Resampling.BILINEAR, "bicubic": Image.Resampling.BICUBIC}[name]
    except ImportError:
        Image = None
    for f, h, w, oh, ow in cases:
        _announce(f"resize {name} {f}x{h}x{w} -> {oh}x{ow}")
        img = rng.integers(0, 256, (f, h, w, 3), dtype=np.uint8)
        got = _resize_gpu(img, oh, ow, name)
        assert got.shape == (f, oh, ow, 3) and got.dtype == np.uint8
        for i in range(f):
            assert np.array_equal(got[i], ro.pil_resize(img[i], oh, ow, name)), (f, h, w, oh, ow, i)
            if Image is not None:
                assert np.array_equal(got[i], np.asarray(Image.fromarray(img[i]).resize((ow, oh), filt)))


def test_resample_pass_with_windows_of_the_callers_own():
    """mvit_resample_u8 takes any windows, not only those of a resize: a mirrored pass (output x reads the inputs
    around in_len - 1 - x, so window starts decrease with x and no LDS span covers a work-group's windows) against numpy."""
    import ctypes as C

    from mi355_vit import _lib

    _announce("resample with mirrored windows")
    rng = np.random.default_rng(21)
    outer, in_len, out_len, inner, ksize = 37, 300, 280, 3, 3
    src = rng.integers(0, 256, (outer, in_len, inner), dtype=np.uint8)
    bounds = np.zeros((out_len, 2), dtype=np.int32)
    kk = np.zeros((out_len, ksize), dtype=np.int32)
    for x in range(out_len):
        c = in_len - 2 - x
        bounds[x] = (c - 1, 3) if c >= 1 else (0, 2)
        kk[x, : bounds[x, 1]] = ((1 << 20), (1 << 21), (1 << 20)) if c >= 1 else ((1 << 21), (1 << 21))
    ref = np.empty((outer, out_len, inner), dtype=np.uint8)
    for x in range(out_len):
        lo, n = bounds[x]
        acc = (1 << 21) + (src[:, lo : lo + n, :].astype(np.int64) * kk[x, :n, None]).sum(axis=1)
        ref[:, x, :] = np.clip(acc >> 22, 0, 255)
    d_src, d_b, d_k = (torch.from_numpy(a).to(DEV) for a in (src, bounds, kk))
    d_dst = torch.zeros(outer, out_len, inner, dtype=torch.uint8, device=DEV)
    rc = _lib.load().mvit_resample_u8(d_src.data_ptr(), d_dst.data_ptr(), outer, in_len, out_len, inner, d_b.data_ptr(), d_k.data_ptr(), ksize,
                                      torch.cuda.current_stream().cuda_stream)
    _lib.check(rc, "mvit_resample_u8")
    torch.cuda.synchronize()
    assert np.array_equal(d_dst.cpu().numpy(), ref)


def test_resize_large_image_against_pillow_and_the_whole_input_chain():
    """A 2,000 x 3,000 photograph-sized image through smart_resize -> bicubic resize -> patchify on the GPU equals the
    same chain on the CPU (Pillow resize where installed, else the oracle; oracle patchify), bit for bit in float32."""
    from oracle import resize_oracle as ro
    from mi355_vit import pixels as P

    _announce("resize 2000x3000 + patchify chain")
    rng = np.random.default_rng(12)
    # smooth content plus noise, so that neighbouring pixels are correlated like in a photograph
    base = rng.integers(0, 256, (1, 50, 75, 3), dtype=np.uint8)
    big = np.clip(np.kron(base, np.ones((1, 40, 40, 1))) + rng.integers(-20, 21, (1, 2000, 3000, 3)), 0, 255).astype(np.uint8)
    th, tw = P.smart_resize(2000, 3000)
    assert (th, tw) == ro.smart_resize(2000, 3000) and th % 28 == 0 and tw % 28 == 0
    got = _resize_gpu(big, th, tw, "bicubic")
    try:
        from PIL import Image
        ref = np.asarray(Image.fromarray(big[0]).resize((tw, th), Image.Resampling.BICUBIC))[None]
    except ImportError:
        ref = ro.pil_resize(big[0], th, tw, "bicubic")[None]
    assert np.array_equal(got, ref)
    pv, grid = P.preprocess([torch.from_numpy(big).to(DEV)])
    torch.cuda.synchronize()
    ref_pv, ref_grid = po.patchify_batch([ref])
    assert grid.tolist() == ref_grid.tolist() == [[1, th // 14, tw // 14]]
    assert np.array_equal(pv.cpu().numpy().view(np.uint32), ref_pv.view(np.uint32))


def test_resize_rejects_what_it_cannot_do():
    from mi355_vit.pixels import resize_frames

    x = torch.zeros(1, 28, 28, 3, dtype=torch.uint8, device=DEV)
    with pytest.raises(ValueError):
        resize_frames(x.float(), 28, 28)
    with pytest.raises(ValueError):
        resize_frames(x, 0, 28)
    with pytest.raises(ValueError):
        resize_frames(x, 28, 56, "lanczos")
    with pytest.raises(RuntimeError):
        resize_frames(x.cpu(), 56, 56)
    same = resize_frames(x, 28, 28)
    assert same.data_ptr() != x.data_ptr() and torch.equal(same, x)
