"""A GGUF file writer for the tests, written from the published format description
(ggml/docs/gguf.md) and independent of the reader under test: little-endian, header
(magic, version, tensor count, key/value count), key/value pairs, tensor infos, padding to the
alignment, tensor data with each tensor's offset a multiple of the alignment."""
from __future__ import annotations

import struct

import numpy as np

U8, I8, U16, I16, U32, I32, F32, BOOL, STRING, ARRAY, U64, I64, F64 = range(13)
_FMT = {U8: "<B", I8: "<b", U16: "<H", I16: "<h", U32: "<I", I32: "<i", F32: "<f", BOOL: "<?",
        U64: "<Q", I64: "<q", F64: "<d"}


def _string(s: str | bytes) -> bytes:
    b = s.encode("utf-8") if isinstance(s, str) else s
    return struct.pack("<Q", len(b)) + b


def _value(vtype: int, v) -> bytes:
    if vtype in _FMT:
        return struct.pack(_FMT[vtype], v)
    if vtype == STRING:
        return _string(v)
    if vtype == ARRAY:
        etype, items = v
        out = struct.pack("<IQ", etype, len(items))
        for it in items:
            out += _value(etype, it)
        return out
    raise ValueError(vtype)


def write_gguf(path, metadata, tensors, version=3, alignment=None, magic=b"GGUF", truncate_data_by=0):
    """metadata: list of (key, value type, value); tensors: list of (name, dims in ne order,
    ggml type id, raw bytes).  Returns {name: absolute file offset of the tensor's data}."""
    metadata = list(metadata)
    if alignment is not None:
        metadata.append(("general.alignment", U32, alignment))
    align = alignment or 32
    head = magic + struct.pack("<IQQ", version, len(tensors), len(metadata))
    for key, vtype, v in metadata:
        head += _string(key) + struct.pack("<I", vtype) + _value(vtype, v)
    infos, data, offsets = b"", b"", {}
    for name, dims, gtype, raw in tensors:
        raw = bytes(np.ascontiguousarray(raw).tobytes()) if not isinstance(raw, (bytes, bytearray)) else bytes(raw)
        data += b"\0" * (-len(data) % align)
        infos += _string(name) + struct.pack("<I", len(dims)) + b"".join(struct.pack("<Q", d) for d in dims)
        infos += struct.pack("<IQ", gtype, len(data))
        offsets[name] = len(data)
        data += raw
    head += infos
    pad = -len(head) % align
    blob = head + b"\0" * pad + data
    if truncate_data_by:
        blob = blob[:-truncate_data_by]
    with open(path, "wb") as f:
        f.write(blob)
    start = len(head) + pad
    return {k: start + v for k, v in offsets.items()}
