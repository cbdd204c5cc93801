"""End-to-end parity of the vision tower (forward, every parameter gradient) against the CPU oracle, and the
VisionTrainer step API on the GPU."""

import copy

import pytest
import torch

from oracle import vit_oracle
from oracle.vit_oracle import OracleConfig, max_rel_err

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _build(cfg_kwargs, seed, dtype):
    from mi355_vit.config import Qwen2_5_VLVisionConfig
    from mi355_vit.modeling import Qwen2_5_VisionTransformerPretrainedModel

    torch.manual_seed(seed)
    model = Qwen2_5_VisionTransformerPretrainedModel(Qwen2_5_VLVisionConfig(**cfg_kwargs))
    model.to(dtype)
    return model


def _oracle_cfg(kw):
    return OracleConfig(**{k: v for k, v in kw.items() if k in OracleConfig.__dataclass_fields__})


def _oracle_run(model_cpu, kw, pixels, grid, gout):
    """fp32 oracle forward/backward on the (possibly bf16-rounded) weights of `model_cpu`."""
    params = {k: v.detach().float().clone().requires_grad_(True) for k, v in model_cpu.state_dict().items()}
    inv_freq = model_cpu.rotary_pos_emb.inv_freq.detach().clone()  # keeps its dtype: bf16 towers build a bf16 table
    out = vit_oracle.tower_forward(pixels.float(), grid, params, _oracle_cfg(kw), inv_freq=inv_freq)
    out.backward(gout.float())
    return out.detach(), {k: p.grad for k, p in params.items()}


def _run_gpu(model, pixels, grid, gout):
    model.to(DEV).train()
    model.zero_grad(set_to_none=True)
    out = model(hidden_states=pixels.to(DEV), grid_thw=grid.to(DEV))
    out.backward(gout.to(device=DEV, dtype=out.dtype))
    return out.detach(), {n: p.grad.detach() for n, p in model.named_parameters()}


CFG1 = dict(depth=4, hidden_size=1280, intermediate_size=3420, num_heads=16, out_hidden_size=2048, fullatt_block_indexes=[3])


def test_config1_fp32_parity():
    """Benchmark configuration 1: reduced tower, fp32, 2 images of 224x224; outputs and all gradients within 1e-4."""
    print("[case] config-1 fp32 tower", flush=True)
    model = _build(CFG1, 0, torch.float32)
    g = torch.Generator().manual_seed(0)
    grid = torch.tensor([[1, 16, 16], [1, 16, 16]])
    pixels = torch.randn(512, 1176, generator=g)
    gout = torch.randn(128, 2048, generator=g)
    ref_out, ref_grads = _oracle_run(copy.deepcopy(model), CFG1, pixels, grid, gout)
    out, grads = _run_gpu(model, pixels, grid, gout)
    assert out.shape == (128, 2048) and out.dtype == torch.float32
    assert max_rel_err(out, ref_out) < 1e-4
    worst = max((max_rel_err(grads[k], ref_grads[k]), k) for k in ref_grads)
    assert worst[0] < 1e-4, worst
    assert set(grads) == set(ref_grads)


@pytest.mark.parametrize("checkpoint", [False, True])
def test_small_ragged_tower_bf16_parity(checkpoint):
    """Ragged images + a video, windows with edge remainders, bf16 kernels vs the fp32 oracle on the same bf16 weights."""
    print(f"[case] bf16 ragged tower checkpoint={checkpoint}", flush=True)
    kw = dict(depth=3, hidden_size=1280, intermediate_size=3420, num_heads=16, out_hidden_size=512, fullatt_block_indexes=[1])
    model = _build(kw, 1, torch.bfloat16)
    if checkpoint:
        model.gradient_checkpointing_enable()
    g = torch.Generator().manual_seed(1)
    grid = torch.tensor([[1, 18, 22], [2, 8, 12], [1, 34, 16]])
    S = int((grid[:, 0] * grid[:, 1] * grid[:, 2]).sum())
    pixels = torch.randn(S, 1176, generator=g).to(torch.bfloat16)
    gout = torch.randn(S // 4, 512, generator=g).to(torch.bfloat16)
    ref_out, ref_grads = _oracle_run(copy.deepcopy(model), kw, pixels, grid, gout)
    out, grads = _run_gpu(model, pixels, grid, gout)
    assert out.dtype == torch.bfloat16
    assert max_rel_err(out, ref_out) < 2e-2
    worst = max((max_rel_err(grads[k], ref_grads[k]), k) for k in ref_grads)
    assert worst[0] < 2e-2, worst


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 1e-4), (torch.bfloat16, 2e-2)])
def test_smallest_images_parity(dtype, tol):
    """The smallest inputs the model takes: one 28 x 28 image (4 patches, one merged token: every GEMM has 4 rows, every
    attention segment 4 tokens) alone and beside a 2-frame video of the same size and a 28 x 56 image, against the oracle."""
    kw = dict(depth=2, hidden_size=256, intermediate_size=300, num_heads=8, out_hidden_size=128, fullatt_block_indexes=[1])
    for grid in (torch.tensor([[1, 2, 2]]), torch.tensor([[1, 2, 2], [2, 2, 2], [1, 2, 4]])):
        print(f"[case] smallest images {grid.tolist()} {dtype}", flush=True)
        model = _build(kw, 2, dtype)
        g = torch.Generator().manual_seed(4)
        S = int((grid[:, 0] * grid[:, 1] * grid[:, 2]).sum())
        pixels = torch.randn(S, 1176, generator=g).to(dtype)
        gout = torch.randn(S // 4, 128, generator=g).to(dtype)
        ref_out, ref_grads = _oracle_run(copy.deepcopy(model), kw, pixels, grid, gout)
        out, grads = _run_gpu(model, pixels, grid, gout)
        assert tuple(out.shape) == (S // 4, 128) and max_rel_err(out, ref_out) < tol
        worst = max((max_rel_err(grads[k], ref_grads[k]), k) for k in ref_grads)
        assert worst[0] < tol, worst


def test_checkpointing_gives_identical_gradients():
    kw = dict(depth=2, hidden_size=256, intermediate_size=300, num_heads=8, out_hidden_size=256, window_size=56, fullatt_block_indexes=[1])
    g = torch.Generator().manual_seed(3)
    grid = torch.tensor([[1, 16, 16], [1, 16, 32]])
    pixels = torch.randn(768, 1176, generator=g)
    gout = torch.randn(192, 256, generator=g)
    res = []
    for ck in (False, True):
        model = _build(kw, 5, torch.float32)
        if ck:
            model.gradient_checkpointing_enable()
        res.append(_run_gpu(model, pixels, grid, gout))
    assert torch.equal(res[0][0], res[1][0])
    for k in res[0][1]:
        assert torch.equal(res[0][1][k], res[1][1][k]), k


def test_second_stream_overlap_gives_identical_gradients():
    """Weight / bias gradients computed on the second stream (default) against the single-stream order: the
    kernels are deterministic, so every gradient must be bit-identical; bf16 at a size where a weight-gradient
    GEMM spans many work-groups and uses split-K, and two backward passes so that buffers are recycled."""
    from mi355_vit import ops

    kw = dict(depth=3, hidden_size=512, intermediate_size=1200, num_heads=8, out_hidden_size=256, window_size=56, fullatt_block_indexes=[1])
    g = torch.Generator().manual_seed(11)
    grid = torch.tensor([[1, 32, 48], [1, 40, 28], [2, 16, 16]])
    S = int((grid[:, 0] * grid[:, 1] * grid[:, 2]).sum())
    pixels = torch.randn(S, 1176, generator=g)
    gout = torch.randn(S // 4, 256, generator=g)
    res = []
    old = ops.OVERLAP_WGRAD
    try:
        for overlap in (True, False):
            ops.OVERLAP_WGRAD = overlap
            model = _build(kw, 7, torch.bfloat16)
            _run_gpu(model, pixels, grid, gout)
            for p_ in model.parameters():
                p_.grad = None
            res.append(_run_gpu(model, pixels, grid, gout))
    finally:
        ops.OVERLAP_WGRAD = old
    assert ops.side_stream(torch.device(DEV)) is not None or not old
    assert torch.equal(res[0][0], res[1][0])
    for k in res[0][1]:
        assert torch.equal(res[0][1][k], res[1][1][k]), k


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("checkpoint", [False, True])
def test_one_call_per_block_equals_the_call_by_call_sequence(dtype, checkpoint):
    """mvit_block_fwd / mvit_block_bwd issue a block's launches from inside the library; the sequence issued call by call
    (MVIT_BLOCK_CALLS=0, and what runs while launches are being timed) must give the same bits: output and every
    gradient, plain and checkpointed, with the weight gradients on the second stream and in line."""
    from mi355_vit import functional, ops

    kw = dict(depth=3, hidden_size=512, intermediate_size=1200, num_heads=8, out_hidden_size=256, window_size=56, fullatt_block_indexes=[1])
    g = torch.Generator().manual_seed(12)
    grid = torch.tensor([[1, 32, 48], [1, 40, 28], [2, 16, 16]])
    S = int((grid[:, 0] * grid[:, 1] * grid[:, 2]).sum())
    pixels = torch.randn(S, 1176, generator=g)
    gout = torch.randn(S // 4, 256, generator=g)
    res = {}
    old_calls, old_overlap = functional.BLOCK_CALLS, ops.OVERLAP_WGRAD
    try:
        for one_call in (True, False):
            for overlap in (True, False):
                functional.BLOCK_CALLS, ops.OVERLAP_WGRAD = one_call, overlap
                model = _build(kw, 7, dtype)
                if checkpoint:
                    model.gradient_checkpointing_enable()
                _run_gpu(model, pixels, grid, gout)
                for p_ in model.parameters():
                    p_.grad = None
                res[(one_call, overlap)] = _run_gpu(model, pixels, grid, gout)  # second pass: buffers are recycled
    finally:
        functional.BLOCK_CALLS, ops.OVERLAP_WGRAD = old_calls, old_overlap
    ref_out, ref_grads = res[(False, False)]
    assert torch.isfinite(ref_out).all()
    for key, (out, grads) in res.items():
        assert torch.equal(out, ref_out), key
        for k in ref_grads:
            assert torch.equal(grads[k], ref_grads[k]), (key, k)


def test_reference_smoke_shape():
    """The reference's own smoke case (tests/test_ragged_sp_smoke.py:27-98): output [192, 256]."""
    kw = dict(hidden_size=256, num_heads=8, depth=2, patch_size=14, in_channels=3, out_hidden_size=256, spatial_merge_size=2,
              window_size=28, fullatt_block_indexes=[1])
    model = _build(kw, 0, torch.float32).to(DEV).eval()
    grid = torch.tensor([[1, 16, 16], [1, 16, 32]], dtype=torch.int64)
    pixels = torch.randn(768, 1176)
    with torch.no_grad():
        out = model(pixels.to(DEV), grid.to(DEV))
    assert out.shape == (192, 256)
    params = {k: v.detach().float().cpu() for k, v in model.state_dict().items()}
    ref = vit_oracle.tower_forward(pixels, grid, params, _oracle_cfg(kw))
    assert ref.shape == (192, 256)
    assert max_rel_err(out, ref) < 1e-4
    flat = model(pixels.flatten().to(DEV), grid.to(DEV))  # the reference's GPU tests pass a flat tensor
    assert torch.equal(flat.detach(), out)


def _trainer_config(**over):
    cfg = dict(seed=0, model_name="unit-test", parallelism="none", dtype="bfloat16", attention_backend="flash_attention_2",
               activation_checkpointing=False, autocast=True, learning_rate=1e-2, weight_decay=0.01, warmup_ratio=0.0,
               warmup_steps=0, lr_scheduler_type="cosine", num_iterations=10, max_grad_norm=1.0, profile_time=True,
               vision_config=dict(depth=2, hidden_size=256, intermediate_size=300, num_heads=8, out_hidden_size=128, fullatt_block_indexes=[1]),
               synthetic_grids=[[1, 16, 16], [1, 8, 24]])
    cfg.update(over)
    return cfg


def test_trainer_steps_on_gpu():
    from mi355_vit.trainer import VisionTrainer

    tr = VisionTrainer(_trainer_config(), rank=0)
    tr.build_model()
    tr.initialize_trainer()
    tr.zero_grad()
    res = tr.forward_step(iteration=3)
    emb = res["vision_embeddings"]
    M = (16 * 16 + 8 * 24) // 4
    assert emb.shape == (1, M, 128) and emb.dtype == torch.bfloat16 and res["iteration"] == 3 and res["sample_index"] == 0
    assert res["forward_time_ms"] > 0
    before = {n: p.detach().clone() for n, p in tr.model.named_parameters()}
    back = tr.backward_step({"grad": torch.randn(M, 128, device=DEV, dtype=torch.bfloat16)})  # 2-D grad for a 3-D output
    assert back["backward_time_ms"] > 0
    contrib = tr.compute_grad_norm_contribution()
    assert contrib["type"] == "none" and contrib["norm_sq"] > 0
    coeff = tr.optimizer_step(global_grad_norm=contrib["norm_sq"] ** 0.5)
    assert coeff == pytest.approx(min(1.0, 1.0 / (contrib["norm_sq"] ** 0.5 + 1e-6)))
    changed = sum(int(not torch.equal(before[n], p.detach())) for n, p in tr.model.named_parameters())
    assert changed == len(before)
    # packed weights follow the optimizer step: a second forward differs from the first
    res2 = tr.forward_step(iteration=4)
    assert res2["sample_index"] == 1
    tr.backward_step(torch.zeros(1, M, 128, device=DEV, dtype=torch.bfloat16))
    with pytest.raises(RuntimeError, match="No pending vision outputs"):
        tr.backward_step(torch.zeros(1, M, 128, device=DEV))
    tr.forward_step()
    with pytest.raises(ValueError, match="No gradient provided"):
        tr.backward_step(None)
    stats = tr.get_memory_stats()
    assert stats["peak_mb"] >= stats["allocated_mb"] > 0


def test_trainer_batched_five_dimensional_pixel_values():
    """The collated [B, C, T, H, W] input of python/ray/vision.py:732-760: every sample is viewed as consecutive
    1176-value rows, one grid is broadcast to all samples, and the output comes back as [B, tokens per image, hidden];
    gradients of a 3-D output arrive in the same shape."""
    from mi355_vit.trainer import VisionTrainer

    torch.manual_seed(3)
    px = torch.randn(3, 3, 2, 56, 56)  # 16 rows of 1176 values per sample
    batches = [{"pixel_values": px, "image_grid_thw": torch.tensor([1, 4, 4]), "sample_index": torch.tensor([5, 6, 7])},
               {"pixel_values": px.reshape(-1, 1176), "image_grid_thw": torch.tensor([[1, 4, 4]] * 3), "sample_index": torch.tensor([0])}]
    outs = []
    for batch in batches:
        tr = VisionTrainer(_trainer_config(autocast=False), rank=0)
        tr.build_model()
        tr.set_data_iterator([batch])
        tr.initialize_trainer()
        res = tr.forward_step(0)
        outs.append(res["vision_embeddings"])
        if batch["pixel_values"].dim() == 5:
            assert res["sample_index"] == [5, 6, 7] and tuple(outs[0].shape) == (3, 4, 128)
            tr.backward_step(torch.ones(3, 4, 128, device=DEV, dtype=torch.bfloat16))
            assert all(p.grad is not None and torch.isfinite(p.grad).all() for p in tr.model.parameters())
            with pytest.raises(ValueError, match="doesn't match pixel_values batch dimension"):
                tr._model_forward({"pixel_values": px.to(DEV), "image_grid_thw": torch.tensor([[1, 4, 4]] * 2, device=DEV)})
    assert tuple(outs[1].shape) == (1, 12, 128) and torch.equal(outs[0].reshape(1, 12, 128), outs[1])


def test_trainer_fifo_and_checkpoint_roundtrip(tmp_path):
    from mi355_vit.trainer import VisionTrainer

    tr = VisionTrainer(_trainer_config(dtype="float32", activation_checkpointing=True, weight_decay=0.0), rank=0)
    tr.build_model()
    tr.initialize_trainer()
    o1 = tr.forward_step(0)["vision_embeddings"]
    o2 = tr.forward_step(1)["vision_embeddings"]
    assert len(tr._pending_outputs) == 2 and tr._pending_outputs[0] is o1
    tr.backward_step(torch.ones_like(o1))
    assert len(tr._pending_outputs) == 1 and tr._pending_outputs[0] is o2
    tr.backward_step(torch.ones_like(o2))
    path = tr.save_checkpoint(str(tmp_path), epoch=2)
    assert path.endswith("epoch_2/vision/rank_0.pt")
    sd = torch.load(path, weights_only=True, map_location="cpu")["model"]
    assert "blocks.0.attn.q_proj.weight" in sd and "merger.mlp.2.bias" in sd and "rotary_pos_emb.inv_freq" not in sd
    tr.optimizer_step()
    assert tr.load_checkpoint(str(tmp_path), epoch=2)
    for k, v in tr.model.state_dict().items():
        assert torch.equal(v.cpu(), sd[k]), k
    assert not tr.load_checkpoint(str(tmp_path), epoch=9)


@pytest.mark.parametrize("dtype,autocast", [(torch.bfloat16, False), (torch.float32, False), (torch.float32, True)])
def test_forward_after_a_fused_adam_step_uses_the_updated_weights(dtype, autocast):
    """The step writes parameters through raw pointers (no version counter moves): the packed operands the blocks
    read must follow anyway.  Same input before and after one step; the second output must match the oracle run on
    the updated parameters and differ from the first output."""
    from mi355_vit.optim import FusedAdam

    print(f"[case] forward after FusedAdam step {dtype} autocast={autocast}", flush=True)
    kw = dict(depth=2, hidden_size=256, intermediate_size=300, num_heads=8, out_hidden_size=128, fullatt_block_indexes=[1])
    model = _build(kw, 5, dtype).to(DEV).train()
    g = torch.Generator().manual_seed(5)
    grid = torch.tensor([[1, 16, 16], [1, 8, 24]])
    S = 16 * 16 + 8 * 24
    pixels = torch.randn(S, 1176, generator=g).to(DEV)
    gout = torch.randn(S // 4, 128, generator=g).to(DEV)
    # gradients for the block parameters only: a change of the output can then only come from the blocks
    block_params = [p for n, p in model.named_parameters() if n.startswith("blocks.")]
    opt = FusedAdam(block_params, lr=5e-3, weight_decay=0.01)

    def forward():
        with torch.autocast("cuda", dtype=torch.bfloat16, enabled=autocast):
            return model(hidden_states=pixels, grid_thw=grid.to(DEV))

    outs = []
    for step in range(3):
        out = forward()
        outs.append(out.detach().float().cpu())
        model.zero_grad(set_to_none=True)
        out.backward(gout.to(out.dtype))
        for n, p in model.named_parameters():
            if not n.startswith("blocks."):
                p.grad = None
        opt.step()
    final = forward().detach().float().cpu()
    torch.cuda.synchronize()
    assert max_rel_err(final, outs[0]) > 5e-2, "three optimizer steps left the output unchanged: stale operands"
    assert max_rel_err(outs[1], outs[0]) > 1e-2
    low = dtype == torch.bfloat16 or autocast
    cpu = copy.deepcopy(model).cpu()
    params = {k: (v.detach().to(torch.bfloat16).float() if low else v.detach().float()).clone() for k, v in cpu.state_dict().items()}
    inv_freq = cpu.rotary_pos_emb.inv_freq.detach().clone()
    with torch.no_grad():
        ref = vit_oracle.tower_forward(pixels.cpu().float(), grid, params, _oracle_cfg(kw), inv_freq=inv_freq)
    assert max_rel_err(final, ref) < (2e-2 if low else 1e-4)
    # a torch optimizer (in-place torch ops) on the same parameters is followed as well
    sgd = torch.optim.SGD(block_params, lr=0.5)
    out = forward()
    model.zero_grad(set_to_none=True)
    out.backward(gout.to(out.dtype))
    sgd.step()
    after_sgd = forward().detach().float().cpu()
    assert max_rel_err(after_sgd, final) > 1e-2


def test_windowed_block_on_each_sequence_parallel_share_equals_the_unsharded_block():
    """One rank's share of a windowed layer under Ulysses sequence parallelism (modeling:492-581): the pack is cut at
    window boundaries, so a block run on a rank's rows with the rank-local window boundaries and rotary rows needs no
    exchange.  For sp = 4 every rank's output (and input gradient) must equal the matching rows of the unsharded block
    bit for bit."""
    from mi355_vit import ops
    from mi355_vit import sequence_parallel_utils as spu
    from mi355_vit.config import Qwen2_5_VLVisionConfig
    from mi355_vit.modeling import Qwen2_5_VLVisionBlock

    print("[case] windowed block on sp=4 shares", flush=True)
    torch.manual_seed(7)
    cfg = Qwen2_5_VLVisionConfig(depth=1, hidden_size=1280, intermediate_size=3420, num_heads=16, out_hidden_size=256, fullatt_block_indexes=[])
    blk = Qwen2_5_VLVisionBlock(cfg, 0).to(torch.bfloat16).to(DEV)
    grid = torch.tensor([[1, 18, 22], [2, 8, 12], [1, 34, 16], [1, 4, 4]])
    _, cu_w = ops.window_index(grid, 2, 112, 14)
    cu_f = ops.cu_seqlens(grid)
    lengths = (cu_f[1:] - cu_f[:-1]).tolist()
    S = sum(lengths)
    g = torch.Generator().manual_seed(7)
    x = torch.randn(S, 1280, generator=g).to(torch.bfloat16).to(DEV)
    ang = torch.randn(S, 40, generator=g)
    emb = torch.cat((ang, ang), dim=-1)
    cos, sin = emb.cos().to(DEV), emb.sin().to(DEV)
    gy = torch.randn(S, 1280, generator=g).to(torch.bfloat16).to(DEV)

    xf = x.clone().requires_grad_(True)
    y_full = blk(xf, cu_seqlens=cu_w.to(DEV), position_embeddings=(cos, sin))
    y_full.backward(gy)
    outs, dxs, metas = [], [], []
    for r in range(4):
        xr, meta = spu.split_pack_by_sp(x, lengths, r, 4, cu_window_seqlens=cu_w)
        gr, _ = spu.split_pack_by_sp(gy, lengths, r, 4, cu_window_seqlens=cu_w)
        cu_local = spu.rebuild_local_cu_seqlens(meta, use_windows=True)
        cos_r, sin_r, _ = spu.build_local_rope(meta, cos, sin)
        assert int(cu_local[-1]) == xr.shape[0] == cos_r.shape[0]
        xr = xr.clone().requires_grad_(True)
        if xr.shape[0]:
            yr = blk(xr, cu_seqlens=cu_local.to(DEV), position_embeddings=(cos_r, sin_r))
            yr.backward(gr)
            outs.append(yr.detach())
            dxs.append(xr.grad)
        else:
            outs.append(xr.detach())
            dxs.append(torch.zeros_like(xr))
        metas.append(meta)
    lm = [m.local_lengths for m in metas]
    assert torch.equal(spu.gather_rank_packs(outs, lm), y_full.detach())
    assert torch.equal(spu.gather_rank_packs(dxs, lm), xf.grad)
    assert sum(o.shape[0] for o in outs) == S and min(o.shape[0] for o in outs) > 0


def test_a_step_recorded_in_a_hip_graph_replays_bit_identically():
    """The library's launches allocate nothing, wait for nothing and use no stream but the caller's (the eager backward's
    second stream joins through events), so a whole forward and a whole backward can be recorded in HIP graphs.  Three
    replays with different inputs, eager steps and synchronisations between them, each equal to the eager step bit for
    bit (kernel order and arguments are the eager ones)."""
    print("[case] forward and backward recorded in HIP graphs", flush=True)
    kw = dict(depth=3, hidden_size=1280, intermediate_size=3420, num_heads=16, out_hidden_size=512, fullatt_block_indexes=[1])
    model = _build(kw, 5, torch.bfloat16).to(DEV).train()
    model.gradient_checkpointing_enable()
    grid = torch.tensor([[1, 18, 22], [2, 8, 12], [1, 34, 16]])  # a host tensor: planning needs no device read-back
    S = int(grid.prod(dim=1).sum())
    params = list(model.parameters())

    def inputs(seed):
        g = torch.Generator().manual_seed(seed)
        return torch.randn(S, 1176, generator=g).to(torch.bfloat16).to(DEV), torch.randn(S // 4, 512, generator=g).to(torch.bfloat16).to(DEV)

    def eager(px, gout):
        model.zero_grad(set_to_none=True)
        out = model(hidden_states=px, grid_thw=grid)
        out.backward(gout)
        torch.cuda.synchronize()
        return out.detach().clone(), [p.grad.detach().clone() for p in params]

    static_px, static_gout = inputs(0)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):  # plans, packed weights and library handles come into being before the recording
        for _ in range(2):
            torch.autograd.grad(model(hidden_states=static_px, grid_thw=grid), params, static_gout)
    torch.cuda.current_stream().wait_stream(side)
    pool = torch.cuda.graph_pool_handle()
    fwd, bwd = torch.cuda.CUDAGraph(), torch.cuda.CUDAGraph()
    with torch.cuda.graph(fwd, pool=pool):
        static_out = model(hidden_states=static_px, grid_thw=grid)
    with torch.cuda.graph(bwd, pool=pool):
        static_grads = torch.autograd.grad(static_out, params, static_gout)
    for seed in (1, 2, 1):
        px, gout = inputs(seed)
        out_e, grads_e = eager(px, gout)
        static_px.copy_(px)
        static_gout.copy_(gout)
        fwd.replay()
        bwd.replay()
        torch.cuda.synchronize()
        assert torch.equal(static_out.detach(), out_e), f"output, inputs {seed}"
        for i, (a, b) in enumerate(zip(static_grads, grads_e)):
            assert torch.equal(a, b), f"gradient {i}, inputs {seed}"
