"""ctypes binding of libmi355vit.so (the C ABI declared in include/mi355_vit.h).

There is no fallback: if the shared library is missing or a call fails, a ``RuntimeError`` is raised.
"""

from __future__ import annotations

import ctypes as C
from pathlib import Path

LIB_PATH = Path(__file__).resolve().parent / "libmi355vit.so"

F32, BF16 = 0, 1

EPI_NONE, EPI_BIAS, EPI_BIAS_RES, EPI_BIAS_GELU, EPI_SWIGLU, EPI_SWIGLU_BWD, EPI_GELU_BWD, EPI_ACCUM = range(8)

_vp, _i64, _i32, _f32 = C.c_void_p, C.c_int64, C.c_int, C.c_float


class GemmArgs(C.Structure):
    _fields_ = [
        ("dtype", _i32), ("out_dtype", _i32), ("trans_a", _i32), ("trans_b", _i32), ("epilogue", _i32),
        ("M", _i64), ("N", _i64), ("K", _i64),
        ("A", _vp), ("lda", _i64),
        ("B", _vp), ("B2", _vp), ("ldb", _i64),
        ("bias", _vp), ("bias2", _vp),
        ("C", _vp), ("ldc", _i64),
        ("R", _vp), ("ldr", _i64),
        ("aux", _vp), ("ldaux", _i64), ("aux_off", _i64),
        ("workspace", _vp), ("workspace_bytes", _i64), ("split_k", _i32),
    ]


class BlockArgs(C.Structure):
    """mvit_block_args: the operands of one transformer block for mvit_block_fwd / mvit_block_bwd."""

    _fields_ = (
        [(n, _i32) for n in ("dtype", "grad_dtype", "C", "I", "Ipad", "nheads", "head_dim", "n_seg", "max_seqlen", "skip_attention",
                             "split_k_down", "split_k_gate_up", "split_k_proj", "split_k_qkv")]
        + [(n, _f32) for n in ("eps", "q_lead_scale", "attn_scale")]
        + [("S", _i64)]
        + [(n, _vp) for n in ("norm1", "norm2", "wqkv", "bqkv", "wproj", "bproj", "wgu", "bgu", "wdown", "bdown",
                              "cu", "seg_order", "cos", "sin", "x",
                              "n1", "qkv", "o", "x1", "n2", "gu", "h", "x2", "rstd1", "rstd2", "lse",
                              "dx2", "dx", "dgu", "dn", "dx1", "dqkv",
                              "g_norm1", "g_norm2", "g_wqkv", "g_bqkv", "g_wproj", "g_bproj", "g_wgu", "g_bgu", "g_wdown", "g_bdown",
                              "workspace")]
        + [("workspace_bytes", _i64), ("side_stream", _vp), ("events", _vp * 5)]
    )


class AdamTensor(C.Structure):
    """mvit_adam_tensor: one row of the device-resident tensor table of the multi-tensor optimizer kernels."""

    _fields_ = [
        ("param", _vp), ("grad", _vp), ("exp_avg", _vp), ("exp_avg_sq", _vp),
        ("numel", _i64), ("first_chunk", _i64),
        ("step_size", _f32), ("bias_correction2_sqrt", _f32), ("weight_decay", _f32), ("unused", _f32),
        ("shadow", _vp), ("shadow_cols", _i64), ("shadow_ld", _i64), ("shadow_dtype", _i32), ("unused2", _i32),
    ]


ADAM_CHUNK = 8192
SUMSQ_STATIC_MAX_CHUNKS = 262144


class Image(C.Structure):
    """mvit_image: one image or video of the device-resident table of mvit_patchify."""

    _fields_ = [("pixels", _vp), ("frames", _i32), ("height", _i32), ("width", _i32), ("reserved", _i32), ("first_row", _i64)]


PIXEL_ROW = 1176

# name -> argument types (every function returns int except the two noted below)
PROTOTYPES = {
    "mvit_rot_pos_ids": [_vp, _i64, _i32, _vp],
    "mvit_window_index": [_vp, _i64, _i32, _i32, _i32, _vp, _vp, _i64, _vp],
    "mvit_cu_seqlens": [_vp, _i64, _vp, _i64, _vp],
    "mvit_sp_token_cuts": [_i64, _i32, _vp],
    "mvit_sp_window_cuts": [_i64, _i32, _vp, _i64, _vp, _vp],
    "mvit_rmsnorm_fwd": [_vp, _vp, _vp, _vp, _i64, _i64, _f32, _i32, _vp],
    "mvit_rmsnorm_bwd": [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _i32, _i64, _i64, _i32, _vp],
    "mvit_reduce_partials": [_vp, _i32, _i64, _vp, _i32, _vp],
    "mvit_colsum": [_vp, _i64, _i64, _i64, _vp, _i32, _i32, _vp],
    "mvit_rope": [_vp, _vp, _vp, _i64, _i32, _i32, _i64, _i32, _i32, _vp],
    "mvit_rope_scaled": [_vp, _vp, _vp, _i64, _i32, _i32, _i64, _i32, _i32, C.c_float, _i32, _vp],
    "mvit_gather_rows": [_vp, _vp, _vp, _i64, _i64, _vp],
    "mvit_segment_copy": [_vp, _vp, _vp, _i64, _i64, _i64, _vp],
    "mvit_pad_pack": [_vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i32, C.c_uint32, _vp],
    "mvit_cast2d": [_vp, _i64, _i32, _vp, _i64, _i32, _i64, _i64, _vp],
    "mvit_gemm": [C.POINTER(GemmArgs), _vp],
    "mvit_attn_fwd": [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _i32, _i32, _i64, _i32, _i32, _i64, _i64, _i64, _i64, _f32, _i32, _vp],
    "mvit_image_token_ranks": [_vp, _vp, _i64, _i64, _i64, _vp, _vp, _vp, _vp],
    "mvit_merge_rows": [_vp, _vp, _vp, _vp, _i64, _i64, _i64, _vp],
    "mvit_adam_step": [_vp, _i32, _i64, C.c_double, C.c_double, C.c_double, C.c_double, _i32, _i32, _vp],
    "mvit_grad_sumsq": [_vp, _i32, _i64, _vp, _vp, _i32, _vp],
    "mvit_grad_sumsq_static": [_vp, _i32, _i64, _vp, _i32, _vp],
    "mvit_patchify": [_vp, _i32, _i64, _vp, C.c_double] + [_f32] * 6 + [_i32, _vp],
    "mvit_resample_u8": [_vp, _vp, _i64, _i64, _i64, _i64, _vp, _vp, _i32, _vp],
    "mvit_patch_embed_pack_weight": [_vp, _i32, _i64, _i64, _vp, _vp],
    "mvit_patch_embed_frames": [_vp, _i32, _i64, _vp, _i64, _vp, _i64, _i32, C.c_double] + [_f32] * 6 + [_vp],
    "mvit_block_fwd": [C.POINTER(BlockArgs), _vp],
    "mvit_block_bwd": [C.POINTER(BlockArgs), _vp],
    "mvit_attn_bwd": [_vp] * 10 + [_i64, _vp, _vp] + [_i32, _i32, _i64, _i32, _i32] + [_i64] * 8 + [_f32, _i32, _vp],
}
EXPORTS = sorted(list(PROTOTYPES) + ["mvit_version", "mvit_last_error", "mvit_attn_bwd_delta_elems", "mvit_block_bwd_workspace_bytes"])
HEADER_VERSION = 200  # MVIT_VERSION of include/mi355_vit.h these prototypes were written for

_lib = None


def load() -> C.CDLL:
    """Load the library once; raise if it has not been built."""
    global _lib
    if _lib is None:
        if not LIB_PATH.exists():
            raise RuntimeError(
                f"{LIB_PATH} is missing: the HIP extension has not been built "
                "(run `python -c 'import __graft_entry__ as g; g.build()'`); there is no fallback path."
            )
        lib = C.CDLL(str(LIB_PATH))
        for name, argtypes in PROTOTYPES.items():
            fn = getattr(lib, name)
            fn.argtypes = argtypes
            fn.restype = C.c_int
        lib.mvit_version.argtypes = []
        lib.mvit_version.restype = C.c_int
        lib.mvit_last_error.argtypes = []
        lib.mvit_last_error.restype = C.c_char_p
        lib.mvit_attn_bwd_delta_elems.argtypes = [_i32, _i64, _i32, _i32, _i32]
        lib.mvit_attn_bwd_delta_elems.restype = _i64
        lib.mvit_block_bwd_workspace_bytes.argtypes = [C.POINTER(BlockArgs)]
        lib.mvit_block_bwd_workspace_bytes.restype = _i64
        if lib.mvit_version() != HEADER_VERSION:
            raise RuntimeError(f"{LIB_PATH} reports interface version {lib.mvit_version()}, these bindings are written for {HEADER_VERSION}: rebuild the library")
        _lib = lib
    return _lib


class Unsupported(RuntimeError):
    """MVIT_ERR_UNSUPPORTED: the library has no kernel for this case (arguments were well-formed)."""


def check(rc: int, what: str) -> None:
    if rc != 0:
        msg = load().mvit_last_error().decode("utf-8", "replace")
        raise (Unsupported if rc == -3 else RuntimeError)(f"{what} failed (code {rc}): {msg}")
