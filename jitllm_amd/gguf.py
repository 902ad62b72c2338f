"""GGUF files through the C ABI: metadata, tensor infos, and weights uploaded from the mapped file.

Mirrors the parts of J/format/GGUF.java (``loadGGUFMetadata`` :40-115, ``GGUFTensorInfo`` :520) and
J/model/loader/ModelLoader.java (``loadTornadoTensorNative`` :246-290) that sit between a model
file and the projections: the parsing itself is done by the library (``jl_gguf_*``), so what a
Java caller binds is what is exercised here.
"""
from __future__ import annotations

import ctypes as C
from dataclasses import dataclass

from . import _lib as L
from .ggml import GGMLType
from .runtime import Context, TornadoTensor


@dataclass(frozen=True)
class GGUFTensorInfo:
    """J/format/GGUF.java:520 -- plus the absolute file offset and the byte size."""
    name: str
    dimensions: tuple
    ggml_type: int
    file_offset: int
    nbytes: int


class GGUF:
    def __init__(self, path: str):
        self._lib = L.load()
        h = C.c_void_p()
        L.check(self._lib.jl_gguf_open(str(path).encode(), C.byref(h)))
        self.handle = h
        self.path = str(path)

    def close(self) -> None:
        if self.handle:
            self._lib.jl_gguf_close(self.handle)
        self.handle = None

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    @property
    def version(self) -> int:
        return self._lib.jl_gguf_version(self.handle)

    def getAlignment(self) -> int:
        return self._lib.jl_gguf_alignment(self.handle)

    def getTensorDataOffset(self) -> int:
        return self._lib.jl_gguf_data_offset(self.handle)

    def tensor_count(self) -> int:
        return self._lib.jl_gguf_tensor_count(self.handle)

    def metadata_count(self) -> int:
        return self._lib.jl_gguf_metadata_count(self.handle)

    def tensor_info(self, index: int) -> GGUFTensorInfo:
        name, t, nd = C.c_char_p(), C.c_int(), C.c_int()
        dims = (C.c_int64 * 4)()
        off, nbytes = C.c_int64(), C.c_int64()
        L.check(self._lib.jl_gguf_tensor_info(self.handle, index, C.byref(name), C.byref(t), C.byref(nd),
                                              dims, C.byref(off), C.byref(nbytes)))
        return GGUFTensorInfo(name.value.decode(), tuple(dims[:nd.value]), t.value, off.value, nbytes.value)

    def getTensorInfos(self) -> dict:
        return {ti.name: ti for ti in (self.tensor_info(i) for i in range(self.tensor_count()))}

    def find(self, name: str) -> int:
        return self._lib.jl_gguf_find(self.handle, name.encode())

    def metadata_int(self, key: str) -> int:
        v = C.c_int64()
        L.check(self._lib.jl_gguf_metadata_int(self.handle, key.encode(), C.byref(v)))
        return v.value

    def metadata_float(self, key: str) -> float:
        v = C.c_double()
        L.check(self._lib.jl_gguf_metadata_float(self.handle, key.encode(), C.byref(v)))
        return v.value

    def metadata_string(self, key: str) -> str:
        v, n = C.c_char_p(), C.c_int64()
        L.check(self._lib.jl_gguf_metadata_string(self.handle, key.encode(), C.byref(v), C.byref(n)))
        return C.string_at(v, n.value).decode()

    def metadata_array(self, key: str):
        """(element type id, element count) of an array value."""
        t, n = C.c_int(), C.c_int64()
        L.check(self._lib.jl_gguf_metadata_array(self.handle, key.encode(), C.byref(t), C.byref(n)))
        return t.value, n.value

    def load_weight(self, ctx: Context, name: str) -> TornadoTensor:
        """The tensor's blocks uploaded from the mapped file, as a projection weight."""
        h = C.c_void_p()
        L.check(self._lib.jl_gguf_upload(ctx.handle, self.handle, name.encode(), C.byref(h)))
        info = self.tensor_info(self.find(name))
        return TornadoTensor.adopt(ctx, h, GGMLType(info.ggml_type), info.dimensions[1], info.dimensions[0],
                                   info.nbytes)
