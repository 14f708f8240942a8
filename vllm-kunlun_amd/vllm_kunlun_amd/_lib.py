"""ctypes binding of libkmoe.so (the C ABI declared in include/kmoe.h).

The library is the only compute path: there is no torch or CPU fallback. If it
has not been built, importing this module raises.
"""
from __future__ import annotations

import ctypes as C
import os

import torch

_PKG_DIR = os.path.dirname(os.path.abspath(__file__))
PROJECT_DIR = os.path.dirname(_PKG_DIR)
LIB_PATH = os.path.join(PROJECT_DIR, "lib", "libkmoe.so")

KMOE_ACT_NONE = 0
KMOE_ACT_SWIGLU = 1
KMOE_ACT_SWIGLUOAI = 2
KMOE_SCORE_SOFTMAX = 0
KMOE_SCORE_SIGMOID = 1
KMOE_FMT_INT8 = 0
KMOE_FMT_FP8_BLOCK = 1
KMOE_FMT_BF16 = 2
KMOE_FMT_W4A16 = 3
KMOE_DT_BF16, KMOE_DT_F16 = 0, 1
KMOE_W_ROWMAJOR, KMOE_W_TILED = 0, 1
KMOE_S_ROWMAJOR, KMOE_S_FRAG16 = 0, 1
KMOE_A_ROWMAJOR, KMOE_A_CHUNKED = 0, 1
STAGES = ("routing", "align", "quant1", "gemm1", "quant2", "gemm2", "shared", "combine")

_ERR_KIND = {-1: ValueError, -2: ValueError, -3: NotImplementedError, -4: RuntimeError, -5: RuntimeError}


class GemmI8Args(C.Structure):
    _fields_ = [
        ("a", C.c_void_p), ("lda", C.c_int64), ("a_max", C.c_void_p), ("row_src", C.c_void_p),
        ("src_div", C.c_int32), ("w", C.c_void_p), ("w_max", C.c_void_p), ("lod", C.c_void_p),
        ("E", C.c_int32), ("n", C.c_int32), ("k", C.c_int32), ("rows", C.c_int32),
        ("y", C.c_void_p), ("ldy", C.c_int64), ("acc_out", C.c_void_p), ("act", C.c_int32),
        ("variant", C.c_int32), ("w_layout", C.c_int32), ("a_layout", C.c_int32), ("a_rows", C.c_int32),
        ("w_tail", C.c_void_p), ("w_max_tail", C.c_void_p), ("tail_row0", C.c_int32), ("tail_rows", C.c_int32),
        ("tail_src0", C.c_int32), ("act_dtype", C.c_int32),
        ("rows_hint", C.c_int32),
    ]


class GemmBf16Args(C.Structure):
    _fields_ = [
        ("a", C.c_void_p), ("lda", C.c_int64), ("row_src", C.c_void_p), ("src_div", C.c_int32),
        ("w", C.c_void_p), ("lod", C.c_void_p),
        ("E", C.c_int32), ("n", C.c_int32), ("k", C.c_int32), ("rows", C.c_int32),
        ("y", C.c_void_p), ("ldy", C.c_int64), ("act", C.c_int32), ("variant", C.c_int32),
        ("w_layout", C.c_int32), ("bias", C.c_void_p), ("act_alpha", C.c_float), ("act_limit", C.c_float),
        ("act_dtype", C.c_int32),
        ("rows_hint", C.c_int32),
    ]


class GemmW4Args(C.Structure):
    _fields_ = [
        ("a", C.c_void_p), ("lda", C.c_int64), ("row_src", C.c_void_p), ("src_div", C.c_int32),
        ("w", C.c_void_p), ("w_scale", C.c_void_p), ("group_size", C.c_int32), ("lod", C.c_void_p),
        ("E", C.c_int32), ("n", C.c_int32), ("k", C.c_int32), ("rows", C.c_int32),
        ("y", C.c_void_p), ("ldy", C.c_int64), ("act", C.c_int32), ("variant", C.c_int32),
        ("w_layout", C.c_int32), ("act_dtype", C.c_int32), ("scale_layout", C.c_int32),
        ("rows_hint", C.c_int32),
    ]


class GemmFp8Args(C.Structure):
    _fields_ = [
        ("a", C.c_void_p), ("lda", C.c_int64), ("a_scale", C.c_void_p), ("row_src", C.c_void_p),
        ("src_div", C.c_int32), ("w", C.c_void_p), ("w_scale", C.c_void_p), ("lod", C.c_void_p),
        ("E", C.c_int32), ("n", C.c_int32), ("k", C.c_int32), ("rows", C.c_int32),
        ("y", C.c_void_p), ("ldy", C.c_int64), ("act", C.c_int32), ("variant", C.c_int32),
        ("w_layout", C.c_int32),
        ("w_tail", C.c_void_p), ("w_scale_tail", C.c_void_p),
        ("tail_row0", C.c_int32), ("tail_rows", C.c_int32), ("tail_src0", C.c_int32), ("act_dtype", C.c_int32),
        ("rows_hint", C.c_int32),
    ]


class MoEArgs(C.Structure):
    _fields_ = [
        ("M", C.c_int32), ("H", C.c_int32), ("E", C.c_int32), ("K", C.c_int32), ("I", C.c_int32),
        ("format", C.c_int32), ("scoring", C.c_int32), ("renormalize", C.c_int32), ("n_group", C.c_int32), ("topk_group", C.c_int32),
        ("routed_scale", C.c_float), ("logits", C.c_void_p), ("bias", C.c_void_p),
        ("x", C.c_void_p), ("w13", C.c_void_p), ("w13_max", C.c_void_p), ("w2", C.c_void_p), ("w2_max", C.c_void_p),
        ("I_shared", C.c_int32), ("ws13", C.c_void_p), ("ws13_max", C.c_void_p), ("ws2", C.c_void_p),
        ("ws2_max", C.c_void_p), ("out_scale", C.c_float), ("out", C.c_void_p),
        ("stage_events", C.POINTER(C.c_void_p)), ("w_layout", C.c_int32), ("w_gate", C.c_void_p),
        ("w13_bias", C.c_void_p), ("w2_bias", C.c_void_p), ("activation", C.c_int32), ("act_alpha", C.c_float),
        ("act_limit", C.c_float), ("ws_layout", C.c_int32),
        ("w13_scale", C.c_void_p), ("w2_scale", C.c_void_p), ("group_size", C.c_int32),
        ("act_dtype", C.c_int32), ("shared_scale", C.c_float), ("tile_variant", C.c_int32), ("w_scale_layout", C.c_int32),
        ("E_global", C.c_int32), ("first_expert", C.c_int32),
        ("flags", C.c_int32),
    ]


class MoELayout(C.Structure):
    _fields_ = [(n, C.c_size_t) for n in (
        "total_bytes", "topk_w", "topk_ids", "moe_index", "sorted_src", "expert_m", "lod", "align_ws",
        "xq", "xmax", "act", "actq", "actmax", "down", "sh_lod", "sh_act", "sh_actq", "sh_actmax", "sh_out",
        "codes_chunked", "logit_planes", "n_logit_planes")]


def _load() -> C.CDLL:
    if not os.path.exists(LIB_PATH):
        raise ImportError(
            f"{LIB_PATH} is missing: build it with `make -C {PROJECT_DIR}` (or __graft_entry__.build()). "
            "There is no fallback path.")
    lib = C.CDLL(LIB_PATH)
    vp, i32, i64, f32, sz = C.c_void_p, C.c_int, C.c_int64, C.c_float, C.c_size_t
    sigs = {
        "kmoe_last_error": (C.c_char_p, []),
        "kmoe_version": (C.c_char_p, []),
        "kmoe_trace_kernels": (None, [i32]),
        "kmoe_silu_table": (i32, [vp, i32, vp]),
        "kmoe_clock_probe": (i32, [vp, i32, i32, vp]),
        "kmoe_traced_kernels": (C.c_char_p, []),
        "kmoe_softmax_topk": (i32, [vp, i32, i32, i32, i32, vp, vp, vp]),
        "kmoe_sigmoid_group_topk_norm": (i32, [vp, vp, i32, i32, i32, i32, i32, f32, vp, vp, vp]),
        "kmoe_block_statistic": (i32, [vp, i32, i32, i32, vp, vp]),
        "kmoe_align_workspace_bytes": (sz, [i32, i32]),
        "kmoe_align": (i32, [vp, i32, i32, vp, vp, vp, vp, vp, sz, vp]),
        "kmoe_gather_rows": (i32, [vp, i64, vp, i32, i32, i32, vp, i64, vp]),
        "kmoe_quant_i8_rows": (i32, [vp, i64, i32, i32, vp, i64, vp, vp]),
        "kmoe_quant_i8_rows_chunked": (i32, [vp, i64, i32, i32, vp, vp, vp]),
        "kmoe_tile_weights_i8": (i32, [vp, vp, i32, i32, i32, vp]),
        "kmoe_swigluoai_and_mul": (i32, [vp, i64, i32, i32, f32, f32, vp, i64, vp]),
        "kmoe_dequant_w4_bf16": (i32, [vp, vp, i64, i32, i32, vp, vp]),
        "kmoe_dequant_w4": (i32, [vp, vp, i64, i32, i32, vp, i32, vp]),
        "kmoe_tile_scales_w4": (i32, [vp, vp, i32, i32, i32, vp]),
        "kmoe_align_local": (i32, [vp, i32, i32, i32, vp, vp, vp, vp, vp, sz, vp]),
        "kmoe_scaled_mm_azp_epilogue": (i32, [vp, i64, i32, i32, vp, i32, vp, i32, vp, vp, vp, vp, i64, i32, vp]),
        "kmoe_quant_i8_static": (i32, [vp, i64, i32, i32, vp, vp, vp, i64, i32, vp]),
        "kmoe_quant_i8_rows_azp": (i32, [vp, i64, i32, i32, vp, i64, vp, vp, i32, vp]),
        "kmoe_router_gemm_workspace_bytes": (sz, [i32, i32, i32]),
        "kmoe_router_gemm_bf16": (i32, [vp, i64, vp, i32, i32, i32, vp, i64, vp, sz, vp]),
        "kmoe_quant_fp8_group128": (i32, [vp, i64, i32, i32, vp, i64, vp, vp]),
        "kmoe_quant_fp8_group128_dt": (i32, [vp, i64, i32, i32, vp, i64, vp, i32, vp]),
        "kmoe_grouped_gemm_i8": (i32, [C.POINTER(GemmI8Args), vp]),
        "kmoe_silu_and_mul": (i32, [vp, i64, i32, i32, vp, i64, vp]),
        "kmoe_combine": (i32, [vp, i64, vp, vp, vp, i32, i32, i32, f32, vp, i64, vp, i64, vp]),
        "kmoe_grouped_gemm_bf16": (i32, [C.POINTER(GemmBf16Args), vp]),
        "kmoe_grouped_gemm_w4a16": (i32, [C.POINTER(GemmW4Args), vp]),
        "kmoe_grouped_gemm_fp8_block": (i32, [C.POINTER(GemmFp8Args), vp]),
        "kmoe_moe_workspace_layout": (i32, [C.POINTER(MoEArgs), C.POINTER(MoELayout)]),
        "kmoe_moe_forward": (i32, [C.POINTER(MoEArgs), vp, sz, vp]),
        "kmoe_moe_forward_static": (i32, [C.POINTER(MoEArgs), vp]),
        "kmoe_quant_i8_rows_dt": (i32, [vp, i64, i32, i32, vp, i64, vp, i32, vp]),
        "kmoe_quant_i8_rows_chunked_dt": (i32, [vp, i64, i32, i32, vp, vp, i32, vp]),
        "kmoe_silu_and_mul_dt": (i32, [vp, i64, i32, i32, vp, i64, i32, vp]),
        "kmoe_combine_dt": (i32, [vp, i64, vp, vp, vp, i32, i32, i32, f32, vp, i64, f32, vp, i64, i32, vp]),
        "kmoe_router_gemm": (i32, [vp, i64, vp, i32, i32, i32, vp, i64, vp, sz, i32, vp]),
    }
    for name, (res, args) in sigs.items():
        fn = getattr(lib, name)
        fn.restype = res
        fn.argtypes = args
    return lib


lib = _load()
EXPORTS = (
    "kmoe_last_error", "kmoe_version", "kmoe_softmax_topk", "kmoe_sigmoid_group_topk_norm", "kmoe_block_statistic",
    "kmoe_align_workspace_bytes", "kmoe_align", "kmoe_gather_rows", "kmoe_quant_i8_rows", "kmoe_quant_i8_rows_chunked", "kmoe_tile_weights_i8", "kmoe_quant_fp8_group128", "kmoe_quant_fp8_group128_dt",
    "kmoe_grouped_gemm_i8", "kmoe_grouped_gemm_bf16", "kmoe_grouped_gemm_w4a16", "kmoe_grouped_gemm_fp8_block", "kmoe_silu_and_mul", "kmoe_combine",
    "kmoe_moe_workspace_layout", "kmoe_moe_forward", "kmoe_router_gemm_workspace_bytes", "kmoe_router_gemm_bf16",
    "kmoe_swigluoai_and_mul", "kmoe_dequant_w4_bf16", "kmoe_dequant_w4", "kmoe_moe_forward_static",
    "kmoe_quant_i8_static", "kmoe_quant_i8_rows_azp", "kmoe_tile_scales_w4", "kmoe_scaled_mm_azp_epilogue", "kmoe_align_local",
    "kmoe_quant_i8_rows_dt", "kmoe_quant_i8_rows_chunked_dt", "kmoe_silu_and_mul_dt", "kmoe_combine_dt", "kmoe_router_gemm",
    "kmoe_trace_kernels", "kmoe_traced_kernels", "kmoe_silu_table", "kmoe_clock_probe",
)
STATIC_WORKSPACE_BYTES = 64 << 20
KMOE_FLAG_SIDE_STREAM = 1


def check(rc: int) -> None:
    """Turns a status code into the reference's error convention: a Python exception."""
    if rc != 0:
        msg = lib.kmoe_last_error().decode()
        raise _ERR_KIND.get(rc, RuntimeError)(f"kmoe error {rc}: {msg}")


def ptr(t: torch.Tensor | None):
    """Device address of a tensor (None -> NULL)."""
    return None if t is None else C.c_void_p(t.data_ptr())


def stream():
    """The current torch HIP stream as a hipStream_t."""
    return C.c_void_p(torch.cuda.current_stream().cuda_stream)


def act_dtype(t: torch.Tensor, what: str = "kmoe") -> int:
    """KMOE_DT_* of an activation tensor (bfloat16 or float16; anything else is refused)."""
    if t.dtype == torch.bfloat16:
        return KMOE_DT_BF16
    if t.dtype == torch.float16:
        return KMOE_DT_F16
    raise NotImplementedError(f"{what}: activations must be bfloat16 or float16, got {t.dtype}")


def require_device(*tensors: torch.Tensor | None) -> None:
    for t in tensors:
        if t is not None and not t.is_cuda:
            raise RuntimeError("kmoe ops run on the GPU only; got a tensor on " + str(t.device))


def require_contig(*tensors: torch.Tensor | None) -> None:
    for t in tensors:
        if t is not None and not t.is_contiguous():
            raise ValueError("kmoe ops need contiguous tensors")
