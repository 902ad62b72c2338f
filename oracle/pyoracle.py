"""ctypes view of the CPU oracle (oracle/jitllm_oracle.c).

TEST INFRASTRUCTURE ONLY.  Imported by tests/, by ``__graft_entry__.smoke()`` and by the
``cpu_baseline`` leg of ``bench.py`` -- never by the ``jitllm_amd`` package, whose kernels must
fail loudly rather than fall back to anything here.
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess

import numpy as np

Q4_0, Q8_0, Q4_K, Q5_K, Q6_K = 2, 8, 12, 13, 14
Q4_1, Q5_0, IQ4_XS = 3, 6, 23
DOT_SCALAR, DOT_VEC128, DOT_VEC256 = 0, 128, 256
DOT_Q8ACT = 8   # Q8_0FloatTensor.dotQ8Activation (-Djitllm.quantizeActivation=true), Q8_0 only

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "_build", "libjitllm_oracle.so")


def build(force: bool = False) -> str:
    """Compile the oracle with gcc (oracle/Makefile); returns the path of the shared object."""
    if force or not os.path.exists(_SO):
        args = ["make", "-C", _HERE] + (["-B"] if force else [])
        subprocess.run(args, check=True, stdout=subprocess.DEVNULL)
    return _SO


_u8p = C.POINTER(C.c_uint8)
_i8p = C.POINTER(C.c_int8)
_f32p = C.POINTER(C.c_float)


class _JRandomState(C.Structure):
    _fields_ = [("seed", C.c_int64), ("nng", C.c_double), ("have", C.c_int)]


_lib = None


def lib() -> C.CDLL:
    global _lib
    if _lib is not None:
        return _lib
    L = C.CDLL(build())
    L.jo_block_elems.argtypes = [C.c_int]
    L.jo_block_bytes.argtypes = [C.c_int]
    L.jo_f16_to_f32.argtypes = [C.c_uint16]
    L.jo_f16_to_f32.restype = C.c_float
    L.jo_f32_to_f16.argtypes = [C.c_float]
    L.jo_f32_to_f16.restype = C.c_uint16
    for name in ("jo_get_float", "jo_get_float_alt"):
        f = getattr(L, name)
        f.argtypes = [C.c_int, _u8p, C.c_int64]
        f.restype = C.c_float
    L.jo_dequant.argtypes = [C.c_int, _u8p, C.c_int64, _f32p]
    L.jo_dequant.restype = None
    L.jo_dot.argtypes = [C.c_int, C.c_int, _u8p, C.c_int64, _f32p, C.c_int64, C.c_int64]
    L.jo_dot.restype = C.c_float
    L.jo_matmul.argtypes = [C.c_int, C.c_int, _u8p, _f32p, _f32p, C.c_int, C.c_int, C.c_int]
    L.jo_matmul.restype = None
    L.jo_matmul_batch.argtypes = [C.c_int, C.c_int, _u8p, _f32p, _f32p, C.c_int, C.c_int,
                                  C.c_int, C.c_int]
    L.jo_matmul_batch.restype = None
    L.jo_swiglu.argtypes = [_f32p, _f32p, C.c_int64]
    L.jo_swiglu.restype = None
    L.jo_rms_scale.argtypes = [_f32p, C.c_int64, C.c_float]
    L.jo_rms_scale.restype = C.c_float
    L.jo_rmsnorm.argtypes = [_f32p, _f32p, _f32p, C.c_int64, C.c_float]
    L.jo_rmsnorm.restype = None
    L.jo_batched_rms_apply_f16.argtypes = [_f32p, _f32p, _f32p, C.c_float, C.c_int64, C.c_int64, _f32p, C.c_void_p]
    L.jo_batched_rms_apply_f16.restype = None
    L.jo_argmax.argtypes = [_f32p, C.c_int64]
    L.jo_argmax.restype = C.c_int64
    L.jo_quantize_q8.argtypes = [_f32p, _i8p, _f32p, C.c_int64, C.c_int64]
    L.jo_quantize_q8.restype = None
    L.jo_gemm_int8_block_scaled.argtypes = [C.c_int, _i8p, _f32p, _u8p, _f32p, C.c_int, C.c_int,
                                            C.c_int, C.c_int]
    L.jo_gemm_int8_block_scaled.restype = None
    _i32p = C.POINTER(C.c_int32)
    L.jo_quantize_q8_blocks.argtypes = [_f32p, C.c_int64, _i8p, _f32p, _i32p]
    L.jo_quantize_q8_blocks.restype = None
    L.jo_matmul_q8x.argtypes = [C.c_int, _u8p, _i8p, _f32p, _i32p, _f32p, C.c_int, C.c_int, C.c_int]
    L.jo_matmul_q8x.restype = None
    L.jo_jrandom_init.argtypes = [C.POINTER(_JRandomState), C.c_int64]
    L.jo_jrandom_next_int.argtypes = [C.POINTER(_JRandomState)]
    L.jo_jrandom_next_int.restype = C.c_int32
    L.jo_jrandom_next_int_bound.argtypes = [C.POINTER(_JRandomState), C.c_int32]
    L.jo_jrandom_next_int_bound.restype = C.c_int32
    L.jo_jrandom_next_boolean.argtypes = [C.POINTER(_JRandomState)]
    L.jo_jrandom_next_gaussian.argtypes = [C.POINTER(_JRandomState)]
    L.jo_jrandom_next_gaussian.restype = C.c_double
    L.jo_jrandom_next_bytes.argtypes = [C.POINTER(_JRandomState), _u8p, C.c_int64]
    L.jo_jrandom_next_bytes.restype = None
    L.jo_java_string_hash.argtypes = [C.c_char_p]
    L.jo_java_string_hash.restype = C.c_int32
    L.jo_max_threads.restype = C.c_int
    _lib = L
    return L


def _u8(a: np.ndarray):
    assert a.dtype == np.uint8 and a.flags.c_contiguous
    return a.ctypes.data_as(_u8p)


def _f32(a: np.ndarray):
    assert a.dtype == np.float32 and a.flags.c_contiguous
    return a.ctypes.data_as(_f32p)


def block_elems(t: int) -> int:
    return lib().jo_block_elems(t)


def block_bytes(t: int) -> int:
    return lib().jo_block_bytes(t)


def max_threads() -> int:
    return lib().jo_max_threads()


def f16_to_f32(bits: int) -> np.float32:
    return np.float32(lib().jo_f16_to_f32(int(bits) & 0xFFFF))


def f32_to_f16(v: float) -> int:
    return int(lib().jo_f32_to_f16(float(np.float32(v))))


def get_float(t: int, w: np.ndarray, i: int, alt: bool = False) -> np.float32:
    f = lib().jo_get_float_alt if alt else lib().jo_get_float
    return np.float32(f(t, _u8(w), i))


def dequant(t: int, w: np.ndarray, n: int | None = None) -> np.ndarray:
    if n is None:
        n = w.size // block_bytes(t) * block_elems(t)
    out = np.empty(n, dtype=np.float32)
    lib().jo_dequant(t, _u8(w), n, _f32(out))
    return out


def dequant_alt(t: int, w: np.ndarray) -> np.ndarray:
    n = w.size // block_bytes(t) * block_elems(t)
    f = lib().jo_get_float_alt
    p = _u8(w)
    return np.array([f(t, p, i) for i in range(n)], dtype=np.float32)


def dot(t: int, flavour: int, w: np.ndarray, this_offset: int, x: np.ndarray, that_offset: int,
        size: int) -> np.float32:
    return np.float32(lib().jo_dot(t, flavour, _u8(w), this_offset, _f32(x), that_offset, size))


def matmul(t: int, w: np.ndarray, x: np.ndarray, dim0: int, dim1: int,
           flavour: int = DOT_SCALAR, nthreads: int = 0) -> np.ndarray:
    out = np.empty(dim0, dtype=np.float32)
    lib().jo_matmul(t, flavour, _u8(w), _f32(x), _f32(out), dim0, dim1,
                    nthreads or max_threads())
    return out


def matmul_batch(t: int, w: np.ndarray, X: np.ndarray, dim0: int, dim1: int,
                 flavour: int = DOT_SCALAR, nthreads: int = 0) -> np.ndarray:
    X = np.ascontiguousarray(X, dtype=np.float32)
    context = X.shape[0]
    out = np.empty((context, dim0), dtype=np.float32)
    lib().jo_matmul_batch(t, flavour, _u8(w), _f32(X), _f32(out), context, dim0, dim1,
                          nthreads or max_threads())
    return out


def swiglu(gate: np.ndarray, up: np.ndarray) -> np.ndarray:
    g = np.ascontiguousarray(gate, dtype=np.float32).copy()
    u = np.ascontiguousarray(up, dtype=np.float32)
    lib().jo_swiglu(_f32(g), _f32(u), g.size)
    return g


def rms_scale(x: np.ndarray, eps: float) -> np.float32:
    """CpuOperations.rmsnorm's factor (J/inference/op/CpuOperations.java:60-66)."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    return np.float32(lib().jo_rms_scale(_f32(x), x.size, eps))


def batched_rms_apply_f16(x: np.ndarray, weight: np.ndarray, eps: float, delta: np.ndarray | None = None,
                          updated: list | None = None):
    """batchedRmsReduceParallel + batchedRmsApplyFP16 (TransformerBatchPrefillKernels.java:1480-1510,
    59-72) over the rows of ``x``: (scales [rows] fp32, out [rows x n] fp16).  With ``delta`` the
    residual add of batchedRmsReduceFusedResidual (:1519-1551) comes first; the updated rows are
    appended to ``updated`` when a list is given (``x`` itself is never modified)."""
    x = np.array(x, dtype=np.float32, order="C", copy=True)
    rows, n = x.shape
    d = None if delta is None else np.ascontiguousarray(delta, dtype=np.float32)
    w = np.ascontiguousarray(weight, dtype=np.float32)
    scales = np.empty(rows, dtype=np.float32)
    out = np.empty((rows, n), dtype=np.float16)
    lib().jo_batched_rms_apply_f16(_f32(x), None if d is None else _f32(d), _f32(w), eps, rows, n, _f32(scales),
                                   out.ctypes.data)
    if updated is not None:
        updated.append(x)
    return scales, out


def rmsnorm(x: np.ndarray, weight: np.ndarray, eps: float) -> np.ndarray:
    """out = weight * (ss * x) (J/inference/op/CpuOperations.java:60-72)."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    w = np.ascontiguousarray(weight, dtype=np.float32)
    out = np.empty_like(x)
    lib().jo_rmsnorm(_f32(out), _f32(x), _f32(w), x.size, eps)
    return out


def argmax(x: np.ndarray) -> int:
    """FloatTensor.argmax (J/tensor/standard/FloatTensor.java:168-181)."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    return int(lib().jo_argmax(_f32(x), x.size))


def quantize_q8(x: np.ndarray):
    x = np.ascontiguousarray(x, dtype=np.float32)
    rows, k = x.shape
    q = np.empty((rows, k), dtype=np.int8)
    s = np.empty((rows, k // 32), dtype=np.float32)
    lib().jo_quantize_q8(_f32(x), q.ctypes.data_as(_i8p), _f32(s), rows, k)
    return q, s


def quantize_q8_blocks(x: np.ndarray):
    """quantizeActivationQ8Blocks: (int8 quants [n], float32 scales [n / 32], int32 sums [n / 32])."""
    x = np.ascontiguousarray(x, dtype=np.float32).reshape(-1)
    q = np.empty(x.size, dtype=np.int8)
    s = np.empty(x.size // 32, dtype=np.float32)
    m = np.empty(x.size // 32, dtype=np.int32)
    lib().jo_quantize_q8_blocks(_f32(x), x.size, q.ctypes.data_as(_i8p), _f32(s),
                                m.ctypes.data_as(C.POINTER(C.c_int32)))
    return q, s, m


def matmul_q8x(t: int, w: np.ndarray, q: np.ndarray, scales: np.ndarray, sums: np.ndarray, dim0: int,
               dim1: int, nthreads: int = 0) -> np.ndarray:
    """The packed-integer projection of a quantised activation, one value per weight row."""
    out = np.empty(dim0, dtype=np.float32)
    q = np.ascontiguousarray(q, dtype=np.int8)
    sums = np.ascontiguousarray(sums, dtype=np.int32)
    lib().jo_matmul_q8x(t, _u8(w), q.ctypes.data_as(_i8p), _f32(scales), sums.ctypes.data_as(C.POINTER(C.c_int32)),
                        _f32(out), dim0, dim1, nthreads or max_threads())
    return out


def gemm_int8_block_scaled(t: int, aq: np.ndarray, ascale: np.ndarray, w: np.ndarray, n: int,
                           nthreads: int = 0) -> np.ndarray:
    m, k = aq.shape
    out = np.empty((m, n), dtype=np.float32)
    lib().jo_gemm_int8_block_scaled(t, aq.ctypes.data_as(_i8p), _f32(ascale), _u8(w), _f32(out),
                                    m, n, k, nthreads or max_threads())
    return out


class JavaRandom:
    """java.util.Random, bit for bit (the generator the reference's test fixtures draw from)."""

    def __init__(self, seed: int):
        self._s = _JRandomState()
        # wrap to a signed 64-bit value as a Java long would
        seed &= (1 << 64) - 1
        if seed >= 1 << 63:
            seed -= 1 << 64
        lib().jo_jrandom_init(C.byref(self._s), seed)

    def next_int(self, bound: int | None = None) -> int:
        if bound is None:
            return lib().jo_jrandom_next_int(C.byref(self._s))
        return lib().jo_jrandom_next_int_bound(C.byref(self._s), bound)

    def next_float(self) -> float:
        """``next(24) / (float)(1 << 24)``: the top 24 of the 32 bits ``nextInt()`` would return."""
        return ((self.next_int() & 0xFFFFFFFF) >> 8) / float(1 << 24)

    def next_boolean(self) -> bool:
        return bool(lib().jo_jrandom_next_boolean(C.byref(self._s)))

    def next_gaussian(self) -> float:
        return lib().jo_jrandom_next_gaussian(C.byref(self._s))

    def next_bytes(self, n: int) -> np.ndarray:
        out = np.empty(n, dtype=np.uint8)
        lib().jo_jrandom_next_bytes(C.byref(self._s), _u8(out), n)
        return out


def java_string_hash(s: str) -> int:
    return lib().jo_java_string_hash(s.encode("utf-8"))
