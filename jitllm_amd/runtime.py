"""Host objects over the C ABI: a device context, fp32 device arrays and resident weights.

Names follow the reference's device-side vocabulary: ``FloatArray`` is TornadoVM's fp32 device
array (the ``wrapX`` / ``wrapXb`` / ``wrapHb`` workspace arrays), ``TornadoTensor`` a weight whose
GGUF blocks live on the device unconverted (J/backend/tornado/tensor/TornadoTensor.java:17-101).
"""
from __future__ import annotations

import ctypes as C

import numpy as np

from . import _lib as L
from .ggml import GGMLType


class Context:
    """One device and one stream (jl_context)."""

    def __init__(self, device: int = 0, stream: int | None = None):
        """``stream``: a hipStream_t the caller owns (an integer handle, e.g. a
        ``torch.cuda.Stream().cuda_stream``); the context then enqueues on it and never destroys it.
        Without one the context makes a stream of its own."""
        self._lib = L.load()
        h = C.c_void_p()
        if stream is None:
            L.check(self._lib.jl_context_create(device, C.byref(h)))
        else:
            L.check(self._lib.jl_context_create_on_stream(device, C.c_void_p(stream), C.byref(h)))
        self.handle = h
        self.device = device

    def close(self) -> None:
        if self.handle:
            self._lib.jl_context_destroy(self.handle)
            self.handle = None

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()

    def sync(self) -> None:
        L.check(self._lib.jl_sync(self.handle))

    @property
    def stream(self) -> int:
        return self._lib.jl_context_stream(self.handle)

    def device_info(self):
        cu = C.c_int()
        name = C.create_string_buffer(128)
        L.check(self._lib.jl_device_info(self.handle, C.byref(cu), name, 128))
        return cu.value, name.value.decode()

    def set_split_k(self, enabled: bool) -> None:
        """False keeps every GEMM of this context whole, as -Djitllm.prefill.splitK=false does in the
        reference (SplitKGemm.java:40-42): a prefill row's sums are then added in one order whatever
        the chunk size."""
        L.check(self._lib.jl_context_set_split_k(self.handle, 1 if enabled else 0))

    # -- arrays --
    def float_array(self, size: int, fill: float | None = None) -> "FloatArray":
        a = FloatArray(self, size)
        if fill is not None:
            a.init(fill)
        return a

    def from_numpy(self, values: np.ndarray) -> "FloatArray":
        values = np.ascontiguousarray(values, dtype=np.float32)
        a = FloatArray(self, values.size)
        a.set(values)
        return a

    def half_array(self, size: int) -> "HalfFloatArray":
        return HalfFloatArray(self, size)

    def half_from_numpy(self, values: np.ndarray) -> "HalfFloatArray":
        a = HalfFloatArray(self, np.asarray(values).size)
        a.set(values)
        return a

    def raw_buffer(self, nbytes: int) -> "DeviceBuffer":
        return DeviceBuffer(self, nbytes)

    # -- weights --
    def load_weight(self, ggml_type, blocks: np.ndarray, rows: int, cols: int) -> "TornadoTensor":
        return TornadoTensor(self, GGMLType(ggml_type), blocks, rows, cols)


class DeviceBuffer:
    """Untyped device memory (jl_malloc / jl_free)."""

    def __init__(self, ctx: Context, nbytes: int):
        self.ctx = ctx
        self.nbytes = int(nbytes)
        p = C.c_void_p()
        L.check(ctx._lib.jl_malloc(ctx.handle, self.nbytes, C.byref(p)))
        self.ptr = p

    def free(self) -> None:
        if self.ptr and self.ctx.handle:
            L.check(self.ctx._lib.jl_free(self.ctx.handle, self.ptr))
        self.ptr = None

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass

    def upload(self, host: np.ndarray, offset: int = 0) -> None:
        host = np.ascontiguousarray(host)
        assert offset + host.nbytes <= self.nbytes
        L.check(self.ctx._lib.jl_upload(self.ctx.handle, self.ptr.value + offset,
                                        host.ctypes.data, host.nbytes))

    def download(self, dtype, count: int, offset: int = 0) -> np.ndarray:
        out = np.empty(count, dtype=dtype)
        assert offset + out.nbytes <= self.nbytes
        L.check(self.ctx._lib.jl_download(self.ctx.handle, out.ctypes.data,
                                          self.ptr.value + offset, out.nbytes))
        return out


class FloatArray(DeviceBuffer):
    """fp32 device array; ``init`` / ``set`` / ``get`` as on TornadoVM's FloatArray."""

    def __init__(self, ctx: Context, size: int):
        super().__init__(ctx, int(size) * 4)
        self.size = int(size)

    def init(self, value: float) -> None:
        L.check(self.ctx._lib.jl_fill_f32(self.ctx.handle, self.ptr, float(value), self.size))

    def set(self, values: np.ndarray) -> None:
        values = np.ascontiguousarray(values, dtype=np.float32).reshape(-1)
        if values.size != self.size:
            raise ValueError(f"{values.size} values for a FloatArray of {self.size}")
        self.upload(values)

    def get(self) -> np.ndarray:
        return self.download(np.float32, self.size)


class HalfFloatArray(DeviceBuffer):
    """IEEE binary16 device array: the activations of the batched prefill (TornadoVM's HalfFloatArray)."""

    def __init__(self, ctx: Context, size: int):
        super().__init__(ctx, int(size) * 2)
        self.size = int(size)

    def set(self, values: np.ndarray) -> None:
        values = np.ascontiguousarray(values, dtype=np.float16).reshape(-1)
        if values.size != self.size:
            raise ValueError(f"{values.size} values for a HalfFloatArray of {self.size}")
        self.upload(values)

    def get(self) -> np.ndarray:
        return self.download(np.float16, self.size)


class TornadoTensor:
    """A weight whose GGUF blocks are resident on the device in the file's layout (jl_weight)."""

    def __init__(self, ctx: Context, ggml_type: GGMLType, blocks: np.ndarray, rows: int, cols: int):
        blocks = np.ascontiguousarray(blocks, dtype=np.uint8).reshape(-1)
        self.ctx = ctx
        self.ggml_type = GGMLType(ggml_type)
        self.rows, self.cols = int(rows), int(cols)
        want = self.ggml_type.byte_size_for(self.rows * self.cols)
        if blocks.size != want:
            raise ValueError(f"{blocks.size} bytes for a {rows}x{cols} {self.ggml_type.name} weight, "
                             f"{want} expected")
        h = C.c_void_p()
        L.check(ctx._lib.jl_weight_upload(ctx.handle, int(self.ggml_type), blocks.ctypes.data,
                                          self.rows, self.cols, C.byref(h)))
        self.handle = h
        self.nbytes = want

    @classmethod
    def adopt(cls, ctx: Context, handle, ggml_type: GGMLType, rows: int, cols: int, nbytes: int) -> "TornadoTensor":
        """Wraps a jl_weight the library created itself (e.g. from a mapped GGUF file)."""
        self = cls.__new__(cls)
        self.ctx, self.ggml_type = ctx, GGMLType(ggml_type)
        self.rows, self.cols, self.handle, self.nbytes = int(rows), int(cols), handle, int(nbytes)
        return self

    def data_type(self) -> GGMLType:
        return self.ggml_type

    def shape(self):
        """GGUF ``ne`` order: dimension 0 is the row length."""
        return (self.cols, self.rows)

    def free(self) -> None:
        if self.handle and self.ctx.handle:
            L.check(self.ctx._lib.jl_weight_free(self.handle))
        self.handle = None

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass

    def dequantize(self) -> np.ndarray:
        """Every element decoded on the device with the host tensor's arithmetic (parity probe)."""
        out = FloatArray(self.ctx, self.rows * self.cols)
        L.check(self.ctx._lib.jl_dequant_f32(self.ctx.handle, self.handle, out.ptr))
        self.ctx.sync()
        res = out.get().reshape(self.rows, self.cols)
        out.free()
        return res


class ResidentCopies:
    """The fp16 copies jl_gemm_resident keeps per set of weights, keyed on the weight objects.

    An entry holds strong references to its ``TornadoTensor`` objects, so neither their identity nor
    their jl_weight address can be handed to another weight while the entry lives; an entry whose
    weights were freed is dropped (its device buffer with it) the next time the cache is asked, so a
    copy never outlives the weights it was decoded from."""

    def __init__(self, context: Context):
        self.context = context
        self._entries: dict = {}

    def lookup(self, weights, swiglu: bool, nbytes_of) -> tuple:
        """(device buffer, int32 state) for this set of weights; ``nbytes_of()`` sizes a new one."""
        dead = [k for k, (ws, _, _) in self._entries.items() if any(not w.handle for w in ws)]
        for k in dead:
            self._entries.pop(k)[1].free()
        if any(not w.handle for w in weights):
            raise ValueError("a freed weight was passed to a resident projection")
        key = tuple(id(w) for w in weights) + (bool(swiglu),)
        if key not in self._entries:
            self._entries[key] = (tuple(weights), DeviceBuffer(self.context, nbytes_of()), C.c_int32(0))
        _, copy, state = self._entries[key]
        return copy, state

    def buffers(self) -> list:
        return [copy for _, copy, _ in self._entries.values()]

    def __len__(self) -> int:
        return len(self._entries)
