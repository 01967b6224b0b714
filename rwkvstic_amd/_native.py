"""ctypes binding of librwkv_hip.so (declarations: include/rwkv_hip.h).

The library is loaded from this directory only; there is no CPU fallback: if
it is missing or a call fails, an exception is raised.
"""
from __future__ import annotations

import ctypes as C
import os

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "librwkv_hip.so")

# every symbol include/rwkv_hip.h declares
EXPORTS = (
    "rwkv_version", "rwkv_last_error",
    "rwkv_mm8_workspace_bytes", "rwkv_mm8_one", "rwkv_mm8_three", "rwkv_wkv_forward_f64",
    "rwkv_mm8_one_static", "rwkv_mm8_one_static_max_bytes",
    "rwkv_mm8_f64_workspace_bytes", "rwkv_mm8_one_f64", "rwkv_mm8_three_f64",
    "rwkv_quantize_u8", "rwkv_packed_bytes", "rwkv_pack_u8", "rwkv_unpack_u8", "rwkv_dequant_packed",
    "rwkv_packed_m16_bytes", "rwkv_pack_m16", "rwkv_unpack_m16",
    "rwkv_mm8_packed", "rwkv_mm8_m16_workspace_bytes", "rwkv_mm8_m16", "rwkv_wkv_f32",
    "rwkv_model_create", "rwkv_model_destroy", "rwkv_model_workspace_bytes",
    "rwkv_model_has_fused_step", "rwkv_model_check", "rwkv_model_set_trace", "rwkv_model_trace_workgroups", "rwkv_model_selftest_timeout", "rwkv_model_time_token_kernel",
    "rwkv_model_forward", "rwkv_model_decode_greedy", "rwkv_argmax_f64",
    "rwkv_sample_token", "rwkv_model_decode_sample",
    "rwkv_gemm8_workspace_bytes", "rwkv_gemm8", "rwkv_gemm8_plan",
    "rwkv_model_batch_workspace_bytes", "rwkv_model_forward_batch",
)


class QMat(C.Structure):
    _fields_ = [("packed", C.c_void_p), ("packed16", C.c_void_p), ("range", C.c_void_p), ("offset", C.c_void_p),
                ("n_in", C.c_int64), ("n_out", C.c_int64)]


class LayerDesc(C.Structure):
    _fields_ = [("ln1_w", C.c_void_p), ("ln1_b", C.c_void_p), ("ln2_w", C.c_void_p), ("ln2_b", C.c_void_p),
                ("att_mix", C.c_void_p), ("ffn_mix", C.c_void_p),
                ("time_decay", C.c_void_p), ("time_first", C.c_void_p),
                ("att_k", QMat), ("att_v", QMat), ("att_r", QMat), ("att_o", QMat),
                ("ffn_k", QMat), ("ffn_r", QMat), ("ffn_v", QMat)]


class ModelDesc(C.Structure):
    _fields_ = [("n_layer", C.c_int64), ("n_embd", C.c_int64), ("n_ffn", C.c_int64), ("n_vocab", C.c_int64),
                ("emb", C.c_void_p), ("ln0_w", C.c_void_p), ("ln0_b", C.c_void_p),
                ("ln_out_w", C.c_void_p), ("ln_out_b", C.c_void_p),
                ("head", QMat), ("layers", C.POINTER(LayerDesc))]


class RwkvHipError(RuntimeError):
    def __init__(self, code: int, message: str):
        super().__init__(f"librwkv_hip error {code}: {message}")
        self.code = code


_lib = None


def lib() -> C.CDLL:
    """Load the shared library once; raise if it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise RuntimeError(
            f"{LIB_PATH} is missing: build it with `python -m rwkvstic_amd.build` "
            "(there is no fallback path)")
    L = C.CDLL(LIB_PATH)
    i64, vp, sz, ci = C.c_int64, C.c_void_p, C.c_size_t, C.c_int
    L.rwkv_version.restype = ci
    L.rwkv_last_error.restype = C.c_char_p
    L.rwkv_mm8_workspace_bytes.restype = sz
    L.rwkv_mm8_workspace_bytes.argtypes = [i64, i64, ci]
    L.rwkv_mm8_one.argtypes = [vp, i64, i64, vp, vp, i64, vp, vp, vp, sz]
    L.rwkv_mm8_one_static.argtypes = [vp, i64, i64, vp, vp, i64, vp, vp]
    L.rwkv_mm8_one_static_max_bytes.restype = sz
    L.rwkv_mm8_one_static_max_bytes.argtypes = []
    L.rwkv_mm8_three.argtypes = [vp, i64, i64, vp, vp, vp, vp, i64, vp, i64, vp, i64,
                                 vp, vp, vp, vp, vp, vp, vp, sz]
    L.rwkv_mm8_f64_workspace_bytes.restype = sz
    L.rwkv_mm8_f64_workspace_bytes.argtypes = [i64, i64, ci]
    L.rwkv_mm8_one_f64.argtypes = [vp, i64, i64, vp, vp, i64, vp, vp, vp, sz]
    L.rwkv_mm8_three_f64.argtypes = [vp, i64, i64, vp, vp, vp, vp, i64, vp, i64, vp, i64,
                                     vp, vp, vp, vp, vp, vp, vp, sz]
    L.rwkv_wkv_forward_f64.argtypes = [vp, i64, i64, i64] + [vp] * 8
    L.rwkv_quantize_u8.argtypes = [vp, vp, i64, i64, vp, vp, vp]
    L.rwkv_packed_bytes.restype = sz
    L.rwkv_packed_bytes.argtypes = [i64, i64]
    L.rwkv_pack_u8.argtypes = [vp, vp, i64, i64, i64, vp]
    L.rwkv_unpack_u8.argtypes = [vp, vp, i64, i64, vp, i64]
    L.rwkv_dequant_packed.argtypes = [vp, vp, vp, vp, i64, i64, vp]
    L.rwkv_packed_m16_bytes.restype = sz
    L.rwkv_packed_m16_bytes.argtypes = [i64, i64]
    L.rwkv_pack_m16.argtypes = [vp, vp, i64, i64, i64, vp]
    L.rwkv_unpack_m16.argtypes = [vp, vp, i64, i64, vp, i64]
    L.rwkv_model_has_fused_step.argtypes = [vp]
    L.rwkv_model_check.argtypes = [vp]
    L.rwkv_model_set_trace.argtypes = [vp, vp]
    L.rwkv_model_trace_workgroups.argtypes = [vp]
    L.rwkv_model_selftest_timeout.argtypes = [vp, vp, vp, vp]
    L.rwkv_model_time_token_kernel.argtypes = [vp, vp, vp, vp, vp, ci, C.POINTER(C.c_float)]
    L.rwkv_mm8_packed.argtypes = [vp, i64, i64, i64, vp, vp, vp, vp, vp, vp, vp]
    L.rwkv_mm8_m16_workspace_bytes.restype = sz
    L.rwkv_mm8_m16_workspace_bytes.argtypes = [i64, i64]
    L.rwkv_mm8_m16.argtypes = [vp, i64, i64, i64, vp, vp, vp, vp, vp, vp, vp, vp, sz]
    L.rwkv_wkv_f32.argtypes = [vp, i64, i64, i64] + [vp] * 8
    L.rwkv_model_create.argtypes = [C.POINTER(ModelDesc), C.POINTER(vp)]
    L.rwkv_model_destroy.argtypes = [vp]
    L.rwkv_model_destroy.restype = None
    L.rwkv_model_workspace_bytes.restype = sz
    L.rwkv_model_workspace_bytes.argtypes = [vp, i64]
    L.rwkv_model_forward.argtypes = [vp, vp, vp, i64, vp, vp, vp, sz]
    L.rwkv_model_decode_greedy.argtypes = [vp, vp, vp, i64, vp, vp, vp, sz]
    L.rwkv_argmax_f64.argtypes = [vp, vp, i64, vp]
    f32, f64, u64 = C.c_float, C.c_double, C.c_uint64
    L.rwkv_sample_token.argtypes = [vp, vp, i64, ci, f32, f32, f64, u64, u64, vp]
    L.rwkv_model_decode_sample.argtypes = [vp, vp, vp, i64, vp, vp, vp, sz, ci, f32, f32, f64, u64, vp, ci, vp, vp]
    L.rwkv_gemm8_workspace_bytes.restype = sz
    L.rwkv_gemm8_workspace_bytes.argtypes = [i64, i64, i64]
    L.rwkv_gemm8.argtypes = [vp, i64, i64, i64, vp, vp, vp, vp, vp, vp, sz]
    L.rwkv_gemm8_plan.argtypes = [i64, i64, i64, ci, C.POINTER(ci * 4), C.POINTER(sz)]
    L.rwkv_model_batch_workspace_bytes.restype = sz
    L.rwkv_model_batch_workspace_bytes.argtypes = [vp, i64]
    L.rwkv_model_forward_batch.argtypes = [vp, vp, vp, i64, vp, vp, vp, sz]
    for name in EXPORTS:
        getattr(L, name)          # AttributeError here means header and library disagree
    _lib = L
    return L


def check(code: int) -> None:
    if code != 0:
        raise RwkvHipError(code, lib().rwkv_last_error().decode())
