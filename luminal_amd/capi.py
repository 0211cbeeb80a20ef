"""ctypes binding of the luminal_hip C ABI (include/luminal_hip.h)."""
from __future__ import annotations

import ctypes as C
import os

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "libluminal_hip.so")

LHIP_OK = 0
LHIP_ERR_NULL_PTR = 1
LHIP_ERR_INVALID_SHAPE = 2
LHIP_ERR_MISALIGNED = 3
LHIP_ERR_HIP = 4
LHIP_ERR_UNSUPPORTED = 5

LHIP_MOE_EXACT, LHIP_MOE_FAST = 0, 1

_vp, _i64, _sz, _int = C.c_void_p, C.c_int64, C.c_size_t, C.c_int

# name -> (restype, argtypes); one entry per declaration in include/luminal_hip.h
SIGNATURES = {
    "lhip_status_string": (C.c_char_p, [C.c_int32]),
    "lhip_last_hip_error": (_int, []),
    "lhip_version": (C.c_char_p, []),
    "lhip_init": (C.c_int32, [_int]),
    "lhip_malloc": (C.c_int32, [C.POINTER(_vp), _sz]),
    "lhip_free": (C.c_int32, [_vp]),
    "lhip_memcpy_h2d": (C.c_int32, [_vp, _vp, _sz, _vp]),
    "lhip_memcpy_d2h": (C.c_int32, [_vp, _vp, _sz, _vp]),
    "lhip_stream_sync": (C.c_int32, [_vp]),
    "lhip_q8_0_raw_nbytes": (_sz, [_i64, _i64]),
    "lhip_q8_0_planar_nbytes": (_sz, [_i64, _i64]),
    "lhip_q8_0_planar_scale_offset": (_sz, [_i64, _i64]),
    "lhip_q8_0_repack": (C.c_int32, [_vp, _vp, _i64, _i64, _vp]),
    "lhip_q8_0_unpack": (C.c_int32, [_vp, _vp, _i64, _i64, _vp]),
    "lhip_q8_0_interleave_rows": (C.c_int32, [_vp, _vp, _vp, _i64, _i64, _vp]),
    "lhip_q8_0_dequant_f32": (C.c_int32, [_vp, _vp, _i64, _i64, _vp]),
    "lhip_q8_0_matmul_f32": (C.c_int32, [_vp, _vp, _vp, _i64, _i64, _i64, _vp]),
    "lhip_q8_0_matmul_f32_cfg": (C.c_int32, [_vp, _vp, _vp, _i64, _i64, _i64, _int, _int, _int, _int, _vp]),
    "lhip_q8_0_gemv_kernel_plan": (C.c_int32, [_i64, _i64, _int, C.c_char_p, C.c_size_t, C.POINTER(C.c_uint32),
                                               C.POINTER(C.c_uint32), C.POINTER(C.c_uint32)]),
    "lhip_decode_program_create": (C.c_int32, [_vp, _int, _i64, _i64, _i64, _i64, C.c_float, _vp, C.POINTER(C.c_void_p)]),
    "lhip_decode_program_run": (C.c_int32, [_vp, _vp]),
    "lhip_decode_program_status": (C.c_int32, [_vp, C.POINTER(C.c_int32)]),
    "lhip_decode_program_destroy": (C.c_int32, [_vp]),
    "lhip_decode_program_trace": (C.c_int32, [_vp, _vp, C.POINTER(C.c_int32)]),
    "lhip_q8_0_matvec_fused_f32": (C.c_int32, [_vp, _vp, _vp, _int, _vp, _i64, _vp, C.c_float, _vp, _int, _vp]),
    "lhip_q8_0_matvec_fused_f32_cfg": (C.c_int32, [_vp, _vp, _vp, _int, _vp, _i64, _vp, C.c_float, _vp, _int, _int, _int,
                                                   _int, _int, _vp]),
    "lhip_q8_0_matmul_bf16": (C.c_int32, [_vp, _vp, _vp, _i64, _i64, _i64, _vp]),
    "lhip_q8_0_matmul_bf16_f32out": (C.c_int32, [_vp, _vp, _vp, _i64, _i64, _i64, _vp]),
    "lhip_q8_0_matmul_bf16_swiglu": (C.c_int32, [_vp, _vp, _vp, _i64, _i64, _i64, _vp]),
    "lhip_q8_0_matmul_bf16_cfg": (C.c_int32, [_vp, _vp, _vp, _i64, _i64, _i64, _int, _vp]),
    "lhip_q8_0_gather_f32": (C.c_int32, [_vp, _vp, _vp, _i64, _i64, _i64, _vp]),
    "lhip_q8_0_matmul_f16": (C.c_int32, [_vp, _vp, _vp, _i64, _i64, _i64, _vp]),
    "lhip_q8_0_matmul_workspace_nbytes": (_sz, [_i64, _i64, _i64]),
    "lhip_q8_0_matmul_f32_ws": (C.c_int32, [_vp, _vp, _vp, _i64, _i64, _i64, _vp, _sz, _vp]),
    "lhip_q8_0_matmul_f16_ws": (C.c_int32, [_vp, _vp, _vp, _i64, _i64, _i64, _vp, _sz, _vp]),
    "lhip_q8_0_matmul_f32_gemm": (C.c_int32, [_vp, _vp, _vp, _i64, _i64, _i64, _vp]),
    "lhip_q8_0_matmul_f16_gemm": (C.c_int32, [_vp, _vp, _vp, _i64, _i64, _i64, _vp]),
    "lhip_q8_0_gather_f16": (C.c_int32, [_vp, _vp, _vp, _i64, _i64, _i64, _vp]),
    "lhip_mxfp4_raw_nbytes": (_sz, [_i64, _i64]),
    "lhip_mxfp4_planar_nbytes": (_sz, [_i64, _i64]),
    "lhip_mxfp4_planar_scale_offset": (_sz, [_i64, _i64]),
    "lhip_mxfp4_repack": (C.c_int32, [_vp, _vp, _i64, _i64, _vp]),
    "lhip_mxfp4_unpack": (C.c_int32, [_vp, _vp, _i64, _i64, _vp]),
    "lhip_mxfp4_dequant_f32": (C.c_int32, [_vp, _vp, _i64, _i64, _vp]),
    "lhip_moe_route_topk": (C.c_int32, [_vp, _vp, _vp, _i64, _i64, _i64, _vp]),
    "lhip_mxfp4_moe_workspace_nbytes": (_sz, [_i64] * 5),
    "lhip_mxfp4_moe_bf16": (C.c_int32, [_vp] * 6 + [_i64] * 5 + [_vp, _vp]),
    "lhip_mxfp4_moe_bf16_mode": (C.c_int32, [_vp] * 6 + [_i64] * 5 + [C.c_int32, _vp, _vp]),
    "lhip_mxfp4_moe_read_intermediates_mode": (C.c_int32, [_vp] * 3 + [_i64] * 5 + [C.c_int32, _vp]),
    "lhip_mxfp4_dequant_bf16": (C.c_int32, [_vp, _vp, _i64, _i64, _vp]),
    "lhip_mxfp4_moe_bf16_static": (C.c_int32, [_vp] * 6 + [_i64] * 5 + [_vp]),
    "lhip_mxfp4_moe_read_intermediates": (C.c_int32, [_vp] * 3 + [_i64] * 5 + [_vp]),
    "lhip_gather_rows_f32": (C.c_int32, [_vp, _vp, _vp, _i64, _i64, _i64, _vp]),
    "lhip_rms_norm_f32": (C.c_int32, [_vp, _vp, _vp, _vp, _vp, _i64, _i64, C.c_float, _vp]),
    "lhip_rms_norm_f32_bf16out": (C.c_int32, [_vp, _vp, _vp, _vp, _vp, _i64, _i64, C.c_float, _vp]),
    "lhip_rope_kv_append_f32": (C.c_int32, [_vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _i64, C.c_float, _vp]),
    "lhip_attention_f32": (C.c_int32, [_vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _i64, _vp]),
    "lhip_attention_f32_bf16out": (C.c_int32, [_vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _i64, _vp]),
    "lhip_attention_bf16": (C.c_int32, [_vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _i64, _vp]),
    "lhip_attention_decode_workspace_nbytes": (C.c_size_t, [_i64, _i64, _i64]),
    "lhip_attention_decode_f32": (C.c_int32, [_vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, C.c_float, _vp, _vp]),
    "lhip_attention_decode_few_ranges_f32": (C.c_int32, [_vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, C.c_float, _vp, _vp]),
    "lhip_attention_decode_partial_f32": (C.c_int32, [_vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, C.c_float, _vp, _vp]),
    "lhip_q8_0_matvec_attn_merge_f32": (C.c_int32, [_vp, _vp, _i64, _i64, _vp, _vp, _i64, _i64, _i64, _i64, _vp, _vp]),
    "lhip_swiglu_f32": (C.c_int32, [_vp, _vp, _i64, _i64, _int, _vp]),
    "lhip_swiglu_f32_bf16out": (C.c_int32, [_vp, _vp, _i64, _i64, _int, _vp]),
    "lhip_cast_f32_to_bf16": (C.c_int32, [_vp, _vp, _i64, _vp]),
    "lhip_cast_bf16_to_f32": (C.c_int32, [_vp, _vp, _i64, _vp]),
    "lhip_add_f32": (C.c_int32, [_vp, _vp, _i64, _vp]),
    "lhip_argmax_f32": (C.c_int32, [_vp, _i64, _vp, _vp, _vp, C.c_int32, _vp]),
    "lhip_argmax_f32_ws": (C.c_int32, [_vp, _i64, _vp, _vp, _vp, C.c_int32, _vp, _vp]),
    "lhip_q8_0_matmul_bf16_workspace_nbytes": (_sz, [_i64, _i64, _i64, C.c_int32]),
    "lhip_q8_0_matmul_bf16_ws": (C.c_int32, [_vp, _vp, _vp, _i64, _i64, _i64, C.c_int32, _vp, _sz, _vp]),
    "lhip_copy_bytes": (C.c_int32, [_vp, _vp, _sz, _vp]),
    "lhip_read_bytes": (C.c_int32, [_vp, _sz, _vp, _vp]),
    "lhip_issue_rate_probe": (C.c_int32, [C.c_int32, C.c_int32, C.c_int32, _vp, _vp]),
}


class LhipError(RuntimeError):
    def __init__(self, status: int, where: str, detail: str = ""):
        self.status = status
        super().__init__(f"{where}: {detail or status}")


_lib = None


class DecodeOp(C.Structure):
    """lhip_decode_op of include/luminal_hip.h."""
    _fields_ = [("type", C.c_int32), ("epilogue", C.c_int32), ("planar", C.c_void_p), ("n", C.c_int64),
                ("k", C.c_int64), ("x", C.c_void_p), ("y", C.c_void_p), ("norm_weight", C.c_void_p),
                ("eps", C.c_float), ("residual", C.c_void_p), ("k_cache", C.c_void_p), ("v_cache", C.c_void_p)]


LHIP_DECODE_MATVEC, LHIP_DECODE_ATTENTION = 0, 1


def load_library(path: str | None = None) -> C.CDLL:
    """Load libluminal_hip.so; there is no fallback if it has not been built."""
    global _lib
    if _lib is not None and path is None:
        return _lib
    p = path or LIB_PATH
    if not os.path.exists(p):
        raise LhipError(-1, "load_library", f"{p} is missing: build it with `python -m luminal_amd.build`")
    lib = C.CDLL(p)
    for name, (res, args) in SIGNATURES.items():
        fn = getattr(lib, name)  # AttributeError if the library does not export it
        fn.restype = res
        fn.argtypes = args
    if path is None:
        _lib = lib
    return lib


def status_string(s: int) -> str:
    return load_library().lhip_status_string(s).decode()


def check(status: int, where: str) -> None:
    if status != LHIP_OK:
        lib = load_library()
        detail = lib.lhip_status_string(status).decode()
        if status == LHIP_ERR_HIP:
            detail += f" (hipError_t {lib.lhip_last_hip_error()})"
        raise LhipError(status, where, detail)
