"""CPU tests: the C-ABI library loads and exports every symbol the header declares; module tree / state-dict
contract; trainer host logic (error paths, clipping, optimizer grouping) without touching a GPU."""

import re
from collections import deque
from pathlib import Path

import pytest
import torch
from torch import nn

ROOT = Path(__file__).resolve().parent.parent


def test_library_exports_every_declared_symbol():
    from mi355_vit import _lib

    header = (ROOT / "include" / "mi355_vit.h").read_text()
    declared = sorted(set(re.findall(r"\b(mvit_[a-z0-9_]+)\s*\(", header)))
    assert declared == _lib.EXPORTS
    lib = _lib.load()
    for name in declared:
        assert hasattr(lib, name), name
    assert lib.mvit_version() == _lib.HEADER_VERSION == int(re.search(r"#define MVIT_VERSION (\d+)", header).group(1))
    assert isinstance(lib.mvit_last_error(), bytes)


def test_attention_backward_refuses_a_short_workspace_and_overlapping_buffers():
    """Host-side argument checks of mvit_attn_bwd: they return before anything is launched, so made-up (aligned,
    never dereferenced) addresses are enough and no GPU is needed."""
    from mi355_vit import _lib

    lib = _lib.load()
    S, H, d = 1024, 16, 80
    C3 = 3 * H * d
    qkv, dqkv, o, do, lse, delta, cu = 0x10000000, 0x20000000, 0x30000000, 0x38000000, 0x40000000, 0x48000000, 0x50000000
    e = 2  # bf16
    need = lib.mvit_attn_bwd_delta_elems(S, S, H, d, _lib.BF16)
    assert need == 3 * H * S and lib.mvit_attn_bwd_delta_elems(64, S, H, d, _lib.BF16) == H * S
    assert lib.mvit_attn_bwd_delta_elems(S, S, H, d, _lib.F32) == H * S

    def call(dq=dqkv, dk=dqkv + H * d * e, dv=dqkv + 2 * H * d * e, n_delta=need, dq_stride=C3):
        # n_seg = 0: the checks run, a call that passes them launches nothing (the addresses are made up)
        return lib.mvit_attn_bwd(qkv, qkv + H * d * e, qkv + 2 * H * d * e, o, do, lse, dq, dk, dv, delta, n_delta, cu, None, 0, S, S, H, d,
                                 C3, C3, C3, H * d, H * d, dq_stride, C3, C3, 1.0, _lib.BF16, None)

    assert call(n_delta=need - 1) == -1 and b"delta workspace" in lib.mvit_last_error()
    assert call(dq=qkv) == -1 and b"dq overlaps q" in lib.mvit_last_error()  # in place on the queries
    assert call(dq=qkv + 8 * e) == -1 and b"dq overlaps" in lib.mvit_last_error()  # shifted by a few columns
    assert call(dk=o, dq_stride=C3) == -1 and b"dk overlaps o" in lib.mvit_last_error()
    assert call() == 0
    # rows interleaved with the inputs in one buffer but on other columns are disjoint and pass the check
    wide_pitch = 2 * C3
    rc = lib.mvit_attn_bwd(qkv, qkv + H * d * e, qkv + 2 * H * d * e, o, do, lse, qkv + C3 * e, qkv + C3 * e + H * d * e, qkv + C3 * e + 2 * H * d * e,
                           delta, need, cu, None, 0, S, S, H, d, wide_pitch, wide_pitch, wide_pitch, H * d, H * d, wide_pitch, wide_pitch, wide_pitch,
                           1.0, _lib.BF16, None)
    assert rc == 0, lib.mvit_last_error()  # no segments: the arguments pass the checks and nothing is launched


def test_gemm_args_struct_matches_header_field_order():
    from mi355_vit import _lib

    header = (ROOT / "include" / "mi355_vit.h").read_text()
    body = header[header.index("typedef struct mvit_gemm_args {") : header.index("} mvit_gemm_args;")]
    fields = re.findall(r"\b(?:int|int64_t|const void\*|void\*)\s+([A-Za-z0-9_, ]+);", body)
    names = [n.strip() for grp in fields for n in grp.split(",")]
    assert names == [f[0] for f in _lib.GemmArgs._fields_]


def test_block_args_struct_matches_header_field_order_and_types():
    import ctypes

    from mi355_vit import _lib

    header = (ROOT / "include" / "mi355_vit.h").read_text()
    body = header[header.index("typedef struct mvit_block_args {") + len("typedef struct mvit_block_args {") : header.index("} mvit_block_args;")]
    want = []
    for stmt in body.split(";"):
        stmt = " ".join(stmt.split())
        if not stmt:
            continue
        m = re.match(r"(const )?(int64_t|int32_t|int|float|void|mvit_stream_t)\b(.*)", stmt)
        assert m, stmt
        base = m.group(2)
        for name in m.group(3).split(","):
            name = name.strip()
            pointer = name.startswith("*") or base == "mvit_stream_t"
            array = re.search(r"\[(\d+)\]", name)
            name = re.sub(r"\[\d+\]", "", name.lstrip("* "))
            if array:
                ctype = ctypes.c_void_p * int(array.group(1))
            elif pointer:
                ctype = ctypes.c_void_p
            else:
                ctype = {"int": ctypes.c_int, "float": ctypes.c_float, "int64_t": ctypes.c_int64}[base]
            want.append((name, ctype))
    got = [(n, t) for n, t in _lib.BlockArgs._fields_]
    assert [n for n, _ in got] == [n for n, _ in want]
    for (n, t), (_, w) in zip(got, want):
        assert ctypes.sizeof(t) == ctypes.sizeof(w) and (t is w or (t._type_ is w._type_ and t._length_ == w._length_) if hasattr(w, "_length_") else t is w), n


def test_ops_refuse_cpu_tensors():
    from mi355_vit import ops

    with pytest.raises(RuntimeError, match="no CPU path"):
        ops.rmsnorm_fwd(torch.randn(4, 8), torch.ones(8), 1e-6)


def test_state_dict_contract_and_default_init():
    from mi355_vit.config import Qwen2_5_VLVisionConfig
    from mi355_vit.modeling import Qwen2_5_VisionTransformerPretrainedModel

    cfg = Qwen2_5_VLVisionConfig(depth=2, hidden_size=64, intermediate_size=36, num_heads=4, out_hidden_size=48, fullatt_block_indexes=[1])
    torch.manual_seed(0)
    m = Qwen2_5_VisionTransformerPretrainedModel(cfg)
    sd = m.state_dict()
    C, I, O = 64, 36, 48
    want = {"patch_embed.proj.weight": (C, 3, 2, 14, 14), "merger.ln_q.weight": (C,), "merger.mlp.0.weight": (4 * C, 4 * C),
            "merger.mlp.0.bias": (4 * C,), "merger.mlp.2.weight": (O, 4 * C), "merger.mlp.2.bias": (O,)}
    for i in range(2):
        b = f"blocks.{i}."
        want.update({b + "norm1.weight": (C,), b + "norm2.weight": (C,)})
        for n in ("q_proj", "k_proj", "v_proj", "proj"):
            want.update({b + f"attn.{n}.weight": (C, C), b + f"attn.{n}.bias": (C,)})
        want.update({b + "mlp.gate_proj.weight": (I, C), b + "mlp.gate_proj.bias": (I,), b + "mlp.up_proj.weight": (I, C),
                     b + "mlp.up_proj.bias": (I,), b + "mlp.down_proj.weight": (C, I), b + "mlp.down_proj.bias": (C,)})
    assert {k: tuple(v.shape) for k, v in sd.items()} == want  # inv_freq is non-persistent
    assert (sd["blocks.0.norm1.weight"] == 1).all()
    # same construction order as the reference => same default init under a seed as plain torch modules built in that order
    torch.manual_seed(0)
    conv = nn.Conv3d(3, C, kernel_size=[2, 14, 14], stride=[2, 14, 14], bias=False)
    q = nn.Linear(C, C)
    assert torch.equal(conv.weight, sd["patch_embed.proj.weight"]) and torch.equal(q.weight, sd["blocks.0.attn.q_proj.weight"])
    # .to(bfloat16) casts the rotary buffer as well (the reference's dtype propagation)
    assert m.to(torch.bfloat16).rotary_pos_emb.inv_freq.dtype == torch.bfloat16
    assert m.spatial_merge_unit == 4 and m.window_size == 112 and len(m.blocks) == 2
    m.gradient_checkpointing_enable()
    assert m.gradient_checkpointing and all(b.gradient_checkpointing for b in m.blocks)
    with pytest.raises(RuntimeError, match="GPU only"):
        m(torch.randn(16, 1176), torch.tensor([[1, 4, 4]]))
    n_params = sum(p.numel() for p in Qwen2_5_VisionTransformerPretrainedModel(Qwen2_5_VLVisionConfig.qwen2_5_vl_tower(depth=1)).parameters())
    per_block = 2 * 1280 + 4 * (1280 * 1280 + 1280) + 2 * (3420 * 1280 + 3420) + 1280 * 3420 + 1280
    assert n_params == 1280 * 1176 + per_block + 1280 + 5120 * 5120 + 5120 + 3584 * 5120 + 3584


def _host_trainer(**over):
    from mi355_vit.trainer import VisionTrainer

    cfg = dict(seed=3, parallelism="none", dtype="bfloat16", learning_rate=1e-3, weight_decay=0.05, warmup_ratio=0.2, warmup_steps=0,
               lr_scheduler_type="linear", num_iterations=10, max_grad_norm=1.0)
    cfg.update(over)
    tr = VisionTrainer(cfg, rank=1)

    class Toy(nn.Module):
        def __init__(self):
            super().__init__()
            self.attn = nn.Linear(4, 4)
            self.norm1 = nn.LayerNorm(4)
            self.ln_q = nn.LayerNorm(4)

    tr.model = Toy()
    return tr


def test_trainer_misuse_errors_and_grad_reshape_on_host():
    tr = _host_trainer()
    with pytest.raises(ValueError, match=r"\[r1\] No gradient provided"):
        tr.backward_step(None)
    with pytest.raises(ValueError, match="No gradient provided"):
        tr.backward_step({"grad": None})
    with pytest.raises(RuntimeError, match="No pending vision outputs available"):
        tr.backward_step(torch.zeros(2, 2))
    x = torch.randn(1, 3, 4, requires_grad=True)
    tr._pending_outputs = deque([x * 2.0])
    tr.backward_step(torch.ones(3, 4))  # 2-D gradient for a 3-D output with batch 1
    assert torch.equal(x.grad, torch.full_like(x, 2.0))
    tr._pending_outputs = deque([torch.randn(2, 3, 4, requires_grad=True) * 1.0])
    with pytest.raises(RuntimeError, match="Dimension mismatch"):
        tr.backward_step(torch.ones(3, 4))
    assert tr.backward_step.__doc__ is None or True


def test_trainer_optimizer_grouping_clip_and_schedule():
    tr = _host_trainer()
    tr._build_optimizer(list(tr.model.parameters()))
    groups = tr.optimizer.param_groups
    assert isinstance(tr.optimizer, torch.optim.Adam) and len(groups) == 2
    assert groups[0]["weight_decay"] == 0.05 and groups[1]["weight_decay"] == 0.0
    assert [tuple(p.shape) for p in groups[0]["params"]] == [(4, 4)]  # only attn.weight decays: bias / norm / ln_ are excluded
    assert len(groups[1]["params"]) == 5
    tr._build_scheduler(10)  # warmup_ratio 0.2 -> 2 warm-up steps, then linear decay
    lrs = []
    for p in tr.model.parameters():
        p.grad = torch.ones_like(p)
    for _ in range(4):
        lrs.append(tr.optimizer.param_groups[0]["lr"])
        tr.optimizer_step()
    assert lrs == pytest.approx([0.0, 0.5e-3, 1e-3, 1e-3 * 7 / 8])
    for p in tr.model.parameters():
        p.grad = torch.ones_like(p)
    contrib = tr.compute_grad_norm_contribution()
    n = sum(p.numel() for p in tr.model.parameters())
    assert contrib == {"type": "none", "norm_sq": pytest.approx(float(n))}
    coeff = tr.optimizer_step(global_grad_norm=4.0)
    assert coeff == pytest.approx(1.0 / (4.0 + 1e-6))
    for p in tr.model.parameters():
        p.grad = torch.ones_like(p)
    tr._clip_gradients(4.0, 1.0)
    assert all(torch.allclose(p.grad, torch.full_like(p, 1.0 / (4.0 + 1e-6))) for p in tr.model.parameters())
    assert tr._clip_gradients(0.5, 1.0) == 1.0
    tr.zero_grad()
    assert all(p.grad is None for p in tr.model.parameters())
    tr2 = _host_trainer(weight_decay=0.0)
    tr2._build_optimizer(list(tr2.model.parameters()))
    assert len(tr2.optimizer.param_groups) == 1 and tr2.optimizer.defaults["foreach"] is False


def test_trainer_config_resolution():
    from mi355_vit.trainer import VisionTrainer, synthetic_batches

    tr = VisionTrainer(dict(seed=0), rank=0)
    assert tr._load_model_config("Qwen/Qwen2.5-VL-7B-Instruct").out_hidden_size == 3584
    assert tr._load_model_config("Qwen/Qwen2.5-VL-3B-Instruct").out_hidden_size == 2048
    assert tr._load_model_config("Qwen/Qwen2.5-VL-32B-Instruct").hidden_size == 1280
    with pytest.raises(ValueError, match="vision_config"):
        tr._load_model_config("somebody/unknown")
    b = next(synthetic_batches([[1, 4, 4], [2, 2, 6]], 0, 1176))
    assert b["pixel_values"].shape == (40, 1176) and b["image_grid_thw"].tolist() == [[1, 4, 4], [2, 2, 6]] and b["sample_index"] == 0
    assert tr._get_torch_dtype("float32") == torch.float32 and tr._get_torch_dtype("nonsense") == torch.bfloat16


def test_segment_lists_are_validated_on_the_host():
    import torch

    from mi355_vit import ops

    ops.check_segments(torch.tensor([0, 4, 4, 9]), 9, 5, torch.tensor([2, 0, 1]))
    for cu, total, mx, order in (([1, 4], 4, 4, None), ([0, 5, 3], 3, 5, None), ([0, 4], 5, 4, None), ([0, 4, 9], 9, 4, None),
                                 ([0, 4, 9], 9, 5, [0, 0]), ([0, 4, 9], 9, 5, [0])):
        try:
            ops.check_segments(torch.tensor(cu), total, mx, None if order is None else torch.tensor(order))
        except ValueError:
            continue
        raise AssertionError(f"accepted {cu}, total {total}, max {mx}, order {order}")


def test_block_parameter_list_follows_the_declared_order():
    """The block hands its 16 parameters to the kernels as a list built from the module dictionaries (no name lookups on
    the hot path): it must be the parameters BLOCK_PARAM_ORDER names, in that order, also after one was replaced."""
    import torch
    from mi355_vit.config import Qwen2_5_VLVisionConfig
    from mi355_vit.functional import BLOCK_PARAM_ORDER
    from mi355_vit.modeling import Qwen2_5_VisionTransformerPretrainedModel

    model = Qwen2_5_VisionTransformerPretrainedModel(Qwen2_5_VLVisionConfig(
        depth=2, hidden_size=64, intermediate_size=100, num_heads=2, out_hidden_size=32, fullatt_block_indexes=[1]))
    for blk in model.blocks:
        assert all(p is blk.get_parameter(n) for p, n in zip(blk._block_params(), BLOCK_PARAM_ORDER, strict=True))
    blk = model.blocks[0]
    blk.attn.proj.weight = torch.nn.Parameter(torch.zeros(64, 64))
    assert blk._block_params()[BLOCK_PARAM_ORDER.index("attn.proj.weight")] is blk.attn.proj.weight


def test_transfer_request_round_trip_and_host_side_choices():
    """python/ray/tensor_transfer.py:101-207 without a GPU: the dictionary form survives a round trip, and a tensor that
    is not on a GPU (or a receiver elsewhere) travels as itself."""
    from mi355_vit.tensor_transfer import TensorTransferRequest, get_physical_gpu_id, prepare_tensor_for_transfer, receive_tensor

    t = torch.arange(6.0).reshape(2, 3)
    req = prepare_tensor_for_transfer(t, ["gpu-a"], "gpu-a")
    assert not req.use_ipc and req.tensor is t and req.ipc_handle is None  # host tensor: never by handle
    back = TensorTransferRequest.from_dict(req.to_dict())
    assert back.tensor is t and back.shape == t.shape and back.dtype == torch.float32 and back.sender_gpu_id == "gpu-a" and not back.use_ipc
    assert receive_tensor(back, "gpu-b") is t
    assert TensorTransferRequest.from_dict({"use_ipc": True, "dtype": "torch.bfloat16"}).dtype == torch.bfloat16
    if not torch.cuda.is_available():
        assert get_physical_gpu_id() == "cpu"


@pytest.mark.parametrize("kind", ["linear", "cosine", "constant", "constant_with_warmup", "polynomial", "inverse_sqrt"])
def test_schedules_equal_the_librarys(kind):
    """The reference builds every schedule with transformers.get_scheduler (python/ray/trainer.py:579-623).  The four
    kinds restated in the trainer must give the library's learning rates step for step; the others are the library's."""
    transformers = pytest.importorskip("transformers")
    tr = _host_trainer(lr_scheduler_type=kind, warmup_ratio=0.0, warmup_steps=3, learning_rate=2e-3)
    tr._build_optimizer(list(tr.model.parameters()))
    tr._build_scheduler(12)
    ref_opt = torch.optim.Adam([torch.nn.Parameter(torch.zeros(1))], lr=2e-3)
    ref = transformers.get_scheduler(name=kind, optimizer=ref_opt, num_warmup_steps=3, num_training_steps=12)
    for _ in range(14):
        assert tr.optimizer.param_groups[0]["lr"] == pytest.approx(ref_opt.param_groups[0]["lr"], rel=1e-12, abs=1e-18)
        tr.optimizer.step()
        tr.scheduler.step()
        ref_opt.step()
        ref.step()


def test_block_entry_points_refuse_malformed_arguments_before_any_launch():
    """mvit_block_fwd / mvit_block_bwd check their struct on the host and return MVIT_ERR_ARG (-1) with a message; nothing
    is launched, so made-up addresses are enough and no GPU is needed."""
    import ctypes

    from mi355_vit import _lib

    lib = _lib.load()
    assert lib.mvit_block_fwd(None, None) == -1 and b"null arguments" in lib.mvit_last_error()
    a = _lib.BlockArgs()
    assert lib.mvit_block_fwd(ctypes.byref(a), None) == -1 and b"bad sizes" in lib.mvit_last_error()
    a.dtype, a.grad_dtype = _lib.BF16, _lib.BF16
    a.S, a.C, a.I, a.Ipad, a.nheads, a.head_dim = 128, 256, 300, 304, 4, 64
    assert lib.mvit_block_fwd(ctypes.byref(a), None) == -1 and b"null weight operand" in lib.mvit_last_error()
    a.head_dim = 60  # heads x head_dim != C
    assert lib.mvit_block_fwd(ctypes.byref(a), None) == -1 and b"bad sizes" in lib.mvit_last_error()
    a.head_dim = 64
    fake = 0x10000000
    for name in ("norm1", "norm2", "wqkv", "bqkv", "wproj", "bproj", "wgu", "bgu", "wdown", "bdown"):
        setattr(a, name, fake)
    assert lib.mvit_block_fwd(ctypes.byref(a), None) == -1 and b"attention geometry missing" in lib.mvit_last_error()
    a.cu, a.cos, a.sin, a.n_seg, a.max_seqlen = fake, fake, fake, 1, 128
    assert lib.mvit_block_fwd(ctypes.byref(a), None) == -1 and b"null activation buffer" in lib.mvit_last_error()
    for name in ("x", "n1", "rstd1", "qkv", "o", "lse", "x1", "n2", "rstd2", "h"):
        setattr(a, name, fake)
    # the backward wants more: saved factors, gradient buffers, slice counts, a workspace of the size it reports
    assert lib.mvit_block_bwd(ctypes.byref(a), None) == -1 and b"null gradient buffer" in lib.mvit_last_error()
    for name in ("gu", "dx2", "dx", "dgu", "dn", "dx1", "dqkv", "g_norm1", "g_norm2", "g_wqkv", "g_bqkv", "g_wproj", "g_bproj", "g_wgu", "g_bgu",
                 "g_wdown", "g_bdown"):
        setattr(a, name, fake)
    assert lib.mvit_block_bwd(ctypes.byref(a), None) == -1 and b"split_k counts" in lib.mvit_last_error()
    a.split_k_down = a.split_k_gate_up = a.split_k_proj = a.split_k_qkv = 2
    need = lib.mvit_block_bwd_workspace_bytes(ctypes.byref(a))
    assert need > 2 * 2 * 304 * 256 * 4  # at least the largest split-K workspace
    a.workspace, a.workspace_bytes = fake, need - 1
    assert lib.mvit_block_bwd(ctypes.byref(a), None) == -1 and b"workspace holds" in lib.mvit_last_error()
    a.workspace_bytes = need
    a.side_stream = fake  # a second stream without its events
    assert lib.mvit_block_bwd(ctypes.byref(a), None) == -1 and b"five events" in lib.mvit_last_error()
    a.S = 0  # an empty block is accepted and does nothing
    a.side_stream = None
    assert lib.mvit_block_fwd(ctypes.byref(a), None) == 0 and lib.mvit_block_bwd(ctypes.byref(a), None) == 0
