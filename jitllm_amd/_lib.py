"""ctypes binding of libjitllm_hip.so -- the same symbols a Java FFM binding would bind.

The library is loaded from ``jitllm_amd/lib/`` (built in-tree by ``jitllm_amd.build``).  There is
no fallback: a missing library or a failing call raises.
"""
from __future__ import annotations

import ctypes as C
import os

from .build import LIB

# include/jitllm_hip.h
JL_OK = 0
JL_ERR_INVALID, JL_ERR_UNSUPPORTED, JL_ERR_HIP, JL_ERR_OOM, JL_ERR_WORKSPACE = -1, -2, -3, -4, -5
JL_STORE, JL_RESIDUAL, JL_SWIGLU = 0, 1, 2
JL_MATH_DEFAULT, JL_MATH_F16, JL_MATH_INT8 = 0, 1, 2
ABI_VERSION = 1

vp = C.c_void_p
i64 = C.c_int64

# every exported symbol: (restype, argtypes)
SYMBOLS = {
    "jl_abi_version": (C.c_int, []),
    "jl_last_error": (C.c_char_p, []),
    "jl_context_create": (C.c_int, [C.c_int, C.POINTER(vp)]),
    "jl_context_create_on_stream": (C.c_int, [C.c_int, vp, C.POINTER(vp)]),
    "jl_context_destroy": (C.c_int, [vp]),
    "jl_sync": (C.c_int, [vp]),
    "jl_context_stream": (vp, [vp]),
    "jl_device_info": (C.c_int, [vp, C.POINTER(C.c_int), C.c_char_p, C.c_size_t]),
    "jl_context_set_split_k": (C.c_int, [vp, C.c_int]),
    "jl_malloc": (C.c_int, [vp, C.c_size_t, C.POINTER(vp)]),
    "jl_free": (C.c_int, [vp, vp]),
    "jl_upload": (C.c_int, [vp, vp, vp, C.c_size_t]),
    "jl_download": (C.c_int, [vp, vp, vp, C.c_size_t]),
    "jl_fill_f32": (C.c_int, [vp, vp, C.c_float, C.c_size_t]),
    "jl_weight_upload": (C.c_int, [vp, C.c_int, vp, i64, i64, C.POINTER(vp)]),
    "jl_weight_wrap": (C.c_int, [vp, C.c_int, vp, i64, i64, C.POINTER(vp)]),
    "jl_weight_free": (C.c_int, [vp]),
    "jl_weight_info": (C.c_int, [vp, C.POINTER(C.c_int), C.POINTER(i64), C.POINTER(i64),
                                 C.POINTER(i64)]),
    "jl_weight_blocks": (vp, [vp]),
    "jl_dequant_f32": (C.c_int, [vp, vp, vp]),
    "jl_gemv": (C.c_int, [vp, vp, vp, vp, C.c_int]),
    "jl_gemv_qkv": (C.c_int, [vp, vp, vp, vp, vp, vp, vp, vp]),
    "jl_gemv_gate_up": (C.c_int, [vp, vp, vp, vp, vp]),
    "jl_swiglu": (C.c_int, [vp, vp, vp, i64]),
    "jl_residual_add": (C.c_int, [vp, vp, vp, i64]),
    "jl_rms_scale": (C.c_int, [vp, vp, i64, C.c_float, vp]),
    "jl_rms_apply": (C.c_int, [vp, vp, vp, vp, i64, vp]),
    "jl_gemv_rms": (C.c_int, [vp, vp, vp, vp, vp, C.c_float, vp, C.c_int]),
    "jl_gemv_qkv_rms": (C.c_int, [vp, vp, vp, vp, vp, vp, vp, C.c_float, vp, vp, vp]),
    "jl_gemv_gate_up_rms": (C.c_int, [vp, vp, vp, vp, vp, C.c_float, vp]),
    "jl_argmax": (C.c_int, [vp, vp, i64, vp]),
    "jl_argmax_rows": (C.c_int, [vp, vp, i64, i64, i64, vp]),
    "jl_gemv_argmax": (C.c_int, [vp, vp, vp, vp, vp, C.c_float, vp, vp]),
    "jl_argmax_static": (C.c_int, [vp, vp, i64, vp]),
    "jl_quantize_q8": (C.c_int, [vp, vp, i64, vp, vp, vp]),
    "jl_rms_quantize_q8": (C.c_int, [vp, vp, vp, vp, i64, vp, vp, vp, vp]),
    "jl_gemv_q8": (C.c_int, [vp, vp, vp, vp, vp, vp, C.c_int]),
    "jl_gemv_qkv_q8": (C.c_int, [vp, vp, vp, vp, vp, vp, vp, vp, vp, vp]),
    "jl_gemv_gate_up_q8": (C.c_int, [vp, vp, vp, vp, vp, vp, vp]),
    "jl_gemm_resident_bytes": (C.c_size_t, [C.POINTER(vp), C.c_int]),
    "jl_gemm_resident": (C.c_int, [vp, C.POINTER(vp), C.c_int, vp, vp, i64, i64, i64, i64, C.c_int, C.c_int,
                                   vp, C.c_size_t, vp, C.c_size_t, C.POINTER(C.c_int32)]),
    "jl_gemm_xf16": (C.c_int, [vp, C.POINTER(vp), C.c_int, vp, vp, C.c_int, i64, i64, i64, i64, C.c_int,
                               vp, C.c_size_t, vp, C.c_size_t, C.POINTER(C.c_int32)]),
    "jl_rms_apply_xf16": (C.c_int, [vp, vp, vp, vp, C.c_float, i64, i64, vp, vp]),
    "jl_gguf_open": (C.c_int, [C.c_char_p, C.POINTER(vp)]),
    "jl_gguf_close": (C.c_int, [vp]),
    "jl_gguf_version": (C.c_int, [vp]),
    "jl_gguf_alignment": (C.c_int, [vp]),
    "jl_gguf_data_offset": (i64, [vp]),
    "jl_gguf_tensor_count": (i64, [vp]),
    "jl_gguf_metadata_count": (i64, [vp]),
    "jl_gguf_find": (i64, [vp, C.c_char_p]),
    "jl_gguf_tensor_info": (C.c_int, [vp, i64, C.POINTER(C.c_char_p), C.POINTER(C.c_int),
                                      C.POINTER(C.c_int), C.POINTER(i64), C.POINTER(i64), C.POINTER(i64)]),
    "jl_gguf_metadata_int": (C.c_int, [vp, C.c_char_p, C.POINTER(i64)]),
    "jl_gguf_metadata_float": (C.c_int, [vp, C.c_char_p, C.POINTER(C.c_double)]),
    "jl_gguf_metadata_string": (C.c_int, [vp, C.c_char_p, C.POINTER(C.c_char_p), C.POINTER(i64)]),
    "jl_gguf_metadata_array": (C.c_int, [vp, C.c_char_p, C.POINTER(C.c_int), C.POINTER(i64)]),
    "jl_gguf_upload": (C.c_int, [vp, vp, C.c_char_p, C.POINTER(vp)]),
    "jl_gemm_workspace_bytes": (C.c_size_t, [i64, i64, i64, C.c_int]),
    "jl_gemm": (C.c_int, [vp, C.POINTER(vp), C.c_int, vp, vp, i64, i64, i64, i64, C.c_int, C.c_int,
                          vp, C.c_size_t]),
}


class JitllmHipError(RuntimeError):
    """A C-ABI call returned a negative status; ``status`` is the jl_status value."""

    def __init__(self, status: int, message: str):
        super().__init__(f"[jl_status {status}] {message}")
        self.status = status


class UnsupportedProjection(JitllmHipError):
    """JL_ERR_UNSUPPORTED: the reference's 'no ... kernel for a ... weight' IllegalStateException."""


_lib = None


def load() -> C.CDLL:
    """Loads the in-tree library and binds every symbol; raises if it is absent."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB):
        raise FileNotFoundError(
            f"{LIB} is not built: run `python -c 'import __graft_entry__ as g; g.build()'` "
            "(there is no CPU fallback for the HIP kernels)")
    lib = C.CDLL(LIB)
    for name, (restype, argtypes) in SYMBOLS.items():
        fn = getattr(lib, name)  # AttributeError names a missing export
        fn.restype = restype
        fn.argtypes = argtypes
    if lib.jl_abi_version() != ABI_VERSION:
        raise RuntimeError(f"libjitllm_hip.so has ABI {lib.jl_abi_version()}, binding wants {ABI_VERSION}")
    _lib = lib
    return lib


def check(status: int) -> None:
    if status == JL_OK:
        return
    msg = load().jl_last_error().decode("utf-8", "replace")
    if status == JL_ERR_UNSUPPORTED:
        raise UnsupportedProjection(status, msg)
    if status == JL_ERR_OOM:
        raise JitllmHipError(status, "GPUL-MEM-001 " + msg)
    raise JitllmHipError(status, msg)
