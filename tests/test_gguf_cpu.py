"""The GGUF reader behind the C ABI, held against files written by an independent writer
(tests/gguf_writer.py).  Parsing is host work: no GPU is needed."""
import numpy as np
import pytest

import gguf_writer as W
from jitllm_amd import synthetic
from jitllm_amd._lib import JitllmHipError
from jitllm_amd.ggml import GGMLType
from jitllm_amd.gguf import GGUF

META = [
    ("general.architecture", W.STRING, "llama"),
    ("general.name", W.STRING, "tiny é中"),           # non-ASCII UTF-8 in a value
    ("llama.block_count", W.U32, 2),
    ("llama.context_length", W.U64, 1 << 33),
    ("llama.attention.layer_norm_rms_epsilon", W.F32, 1e-5),
    ("llama.rope.freq_base", W.F64, 500000.0),
    ("llama.some_i8", W.I8, -7),
    ("llama.some_i16", W.I16, -300),
    ("llama.some_u16", W.U16, 65535),
    ("llama.some_i32", W.I32, -123456),
    ("llama.some_i64", W.I64, -(1 << 40)),
    ("llama.flag", W.BOOL, True),
    ("tokenizer.ggml.tokens", W.ARRAY, (W.STRING, ["<s>", "</s>", "a", "bc", ""])),
    ("tokenizer.ggml.scores", W.ARRAY, (W.F32, [0.0, -1.0, -2.5])),
    ("tokenizer.ggml.token_type", W.ARRAY, (W.I32, [1, 2, 3, 4])),
    ("nested.arrays", W.ARRAY, (W.ARRAY, [(W.U8, [1, 2, 3]), (W.STRING, ["x", "yz"])])),
]


def tensors():
    d, n = 8, 256
    return [
        ("blk.0.attn_q.weight", (n, d), 8, synthetic.weight(GGMLType.Q8_0, d, n, seed=1)),
        ("blk.0.ffn_gate.weight", (n, 2 * d), 2, synthetic.weight(GGMLType.Q4_0, 2 * d, n, seed=2)),
        ("blk.0.ffn_down.weight", (n, d), 12, synthetic.weight(GGMLType.Q4_K, d, n, seed=3)),
        ("blk.0.attn_norm.weight", (n,), 0, np.arange(n, dtype=np.float32)),
        ("token_embd.weight", (n, 3), 14, np.zeros(3 * 210, dtype=np.uint8)),          # Q6_K: 210 B / 256
        ("odd.iq2", (256,), 16, np.zeros(10, dtype=np.uint8)),                         # a type with no geometry
    ]


@pytest.mark.parametrize("version,alignment", [(3, None), (2, None), (3, 64), (3, 4096)])
def test_reader_agrees_with_what_was_written(tmp_path, version, alignment):
    path = tmp_path / "m.gguf"
    ts = tensors()
    where = W.write_gguf(path, META, ts, version=version, alignment=alignment)
    with GGUF(path) as g:
        assert g.version == version
        assert g.getAlignment() == (alignment or 32)
        assert g.getTensorDataOffset() % g.getAlignment() == 0
        assert g.tensor_count() == len(ts)
        assert g.metadata_count() == len(META) + (1 if alignment else 0)
        assert g.metadata_string("general.architecture") == "llama"
        assert g.metadata_string("general.name") == "tiny é中"
        assert g.metadata_int("llama.block_count") == 2
        assert g.metadata_int("llama.context_length") == 1 << 33
        assert g.metadata_float("llama.attention.layer_norm_rms_epsilon") == float(np.float32(1e-5))
        assert g.metadata_float("llama.rope.freq_base") == 500000.0
        assert (g.metadata_int("llama.some_i8"), g.metadata_int("llama.some_i16")) == (-7, -300)
        assert (g.metadata_int("llama.some_u16"), g.metadata_int("llama.some_i32")) == (65535, -123456)
        assert g.metadata_int("llama.some_i64") == -(1 << 40)
        assert g.metadata_int("llama.flag") == 1
        assert g.metadata_array("tokenizer.ggml.tokens") == (W.STRING, 5)
        assert g.metadata_array("tokenizer.ggml.scores") == (W.F32, 3)
        assert g.metadata_array("nested.arrays") == (W.ARRAY, 2)
        infos = g.getTensorInfos()
        raw_file = path.read_bytes()
        for name, dims, gtype, raw in ts:
            ti = infos[name]
            assert (ti.dimensions, ti.ggml_type, ti.file_offset) == (tuple(dims), gtype, where[name])
            assert ti.file_offset % g.getAlignment() == 0
            want = np.ascontiguousarray(raw).tobytes()
            if gtype == 16:
                assert ti.nbytes == -1
            else:
                assert ti.nbytes == len(want)
                assert raw_file[ti.file_offset:ti.file_offset + ti.nbytes] == want
        assert g.find("blk.0.attn_q.weight") == 0 and g.find("no.such.tensor") == -1
        for i, (name, *_rest) in enumerate(ts):     # file order is kept
            assert g.tensor_info(i).name == name


def test_wrong_kinds_and_missing_keys_are_errors(tmp_path):
    path = tmp_path / "m.gguf"
    W.write_gguf(path, META, tensors())
    with GGUF(path) as g:
        with pytest.raises(JitllmHipError, match="no metadata key"):
            g.metadata_int("llama.absent")
        with pytest.raises(JitllmHipError, match="not an integer"):
            g.metadata_int("general.architecture")
        with pytest.raises(JitllmHipError, match="not a string"):
            g.metadata_string("llama.block_count")
        with pytest.raises(JitllmHipError, match="not a float"):
            g.metadata_float("llama.block_count")
        with pytest.raises(JitllmHipError, match="not an array"):
            g.metadata_array("llama.block_count")
        with pytest.raises(JitllmHipError):
            g.tensor_info(99)


def test_files_the_reference_refuses_are_refused_in_its_words(tmp_path):
    bad_magic = tmp_path / "magic.gguf"
    W.write_gguf(bad_magic, META, tensors(), magic=b"GGML")
    with pytest.raises(JitllmHipError, match="unsupported header.magic"):
        GGUF(bad_magic)
    v1 = tmp_path / "v1.gguf"
    W.write_gguf(v1, META, tensors(), version=1)
    with pytest.raises(JitllmHipError, match="unsupported header.version 1"):
        GGUF(v1)
    with pytest.raises(JitllmHipError, match="Model file not found"):
        GGUF(tmp_path / "absent.gguf")
    cut = tmp_path / "cut.gguf"
    W.write_gguf(cut, META, tensors())
    blob = cut.read_bytes()
    cut.write_bytes(blob[:200])                      # ends inside the metadata
    with pytest.raises(JitllmHipError, match="ends early|malformed"):
        GGUF(cut)
    odd = tmp_path / "align.gguf"
    W.write_gguf(odd, META, tensors(), alignment=48)
    with pytest.raises(JitllmHipError, match="not a power of two"):
        GGUF(odd)
    tiny = tmp_path / "tiny.gguf"
    tiny.write_bytes(b"GGUF")
    with pytest.raises(JitllmHipError, match="too short"):
        GGUF(tiny)


def _crafted(tmp_path, name, tensor_count=1, kv=(), offset=0, dims=(256, 8), gtype=8, data=b"\0" * 4096):
    """A file put together by hand so that single header fields can hold hostile values."""
    import struct
    head = b"GGUF" + struct.pack("<IQQ", 3, tensor_count, len(kv))
    for key, vtype, v in kv:
        head += W._string(key) + struct.pack("<I", vtype) + W._value(vtype, v)
    head += W._string("t") + struct.pack("<I", len(dims)) + b"".join(struct.pack("<Q", d) for d in dims)
    head += struct.pack("<IQ", gtype, offset)
    blob = head + b"\0" * (-len(head) % 32) + data
    path = tmp_path / name
    path.write_bytes(blob)
    return path


def _upload_without_context(g, name="t"):
    """jl_gguf_upload reports what is wrong with the file's tensor before it looks at the context,
    so the bounds checks run without a GPU."""
    import ctypes as C
    from jitllm_amd import _lib as L
    h = C.c_void_p()
    L.check(g._lib.jl_gguf_upload(None, g.handle, name.encode(), C.byref(h)))


def test_hostile_header_fields_are_refused_not_followed(tmp_path):
    # a sane file first: the only thing missing is the context
    with GGUF(_crafted(tmp_path, "ok.gguf")) as g:
        assert g.tensor_info(0).nbytes == 8 * 256 // 32 * 34
        with pytest.raises(JitllmHipError, match="null context"):
            _upload_without_context(g)
    # a tensor offset near 2^63: data_offset + offset wraps negative in signed arithmetic
    for off in ((1 << 63) - 40, (1 << 63) - 1, 1 << 63, (1 << 64) - 32, 4096 - 2175):
        with GGUF(_crafted(tmp_path, "far.gguf", offset=off)) as g:
            with pytest.raises(JitllmHipError, match="runs past the end"):
                _upload_without_context(g)
            g.tensor_info(0)         # reporting it must not trap either
    # the last byte of the tensor is the last byte of the file: still inside
    with GGUF(_crafted(tmp_path, "edge.gguf", offset=4096 - 2176)) as g:
        with pytest.raises(JitllmHipError, match="null context"):
            _upload_without_context(g)
    # dimensions whose product overflows 64 bits leave no size to trust
    with GGUF(_crafted(tmp_path, "dims.gguf", dims=(1 << 40, 1 << 40))) as g:
        with pytest.raises(JitllmHipError, match="runs past the end"):
            _upload_without_context(g)
    # general.alignment = 2^32 narrows to 0 in 32 bits (and 0 divides); 2^40 is a power of two too
    for a in (1 << 32, 1 << 40, (1 << 32) + 32):
        with pytest.raises(JitllmHipError, match="general.alignment"):
            GGUF(_crafted(tmp_path, "al.gguf", kv=[("general.alignment", W.U64, a)]))
    # a tensor count that the file could not possibly hold must not size the tensor table
    for count in (1 << 40, 400):
        with pytest.raises(JitllmHipError, match="impossible counts|malformed|end early"):
            GGUF(_crafted(tmp_path, "count.gguf", tensor_count=count))


def test_mutated_files_get_a_status_from_every_call(tmp_path):
    """1 500 seeded mutations of a valid file -- flipped bytes, truncations, inserted bytes, length
    and type fields overwritten with boundary values: opening either fails with a message or gives a
    file every accessor answers with a status; a tensor is never uploaded without a context, and
    never before the file's own faults are reported."""
    import ctypes as C
    import struct

    from jitllm_amd import _lib as L
    lib = L.load()
    rng = np.random.default_rng(20261124)
    base = tmp_path / "base.gguf"
    W.write_gguf(base, META, tensors())
    blob = bytearray(base.read_bytes())
    keys = [k.encode() for k, _, _ in META] + [b"general.alignment", b"no.such.key"]
    big = [2 ** 64 - 1, 2 ** 63, 2 ** 62, 2 ** 32, 2 ** 31, len(blob), len(blob) + 1, 0]
    small = [2 ** 32 - 1, 2 ** 31, 13, 12, 9, 8, 5, 0]
    opened = 0
    path = tmp_path / "mutated.gguf"
    for case in range(1500):
        b = bytearray(blob)
        kind = int(rng.integers(0, 5))
        if kind == 0:
            for _ in range(int(rng.integers(1, 4))):
                b[int(rng.integers(0, len(b)))] = int(rng.integers(0, 256))
        elif kind == 1:
            b = b[:int(rng.integers(0, len(b)))]
        elif kind == 2:
            at = int(rng.integers(0, len(b) - 8))
            b[at:at + 8] = struct.pack("<Q", big[int(rng.integers(0, 8))])
        elif kind == 3:
            at = int(rng.integers(0, len(b) - 4))
            b[at:at + 4] = struct.pack("<I", small[int(rng.integers(0, 8))])
        else:
            at = int(rng.integers(0, len(b)))
            b[at:at] = bytes(rng.integers(0, 256, int(rng.integers(1, 40)), dtype=np.uint8))
        path.write_bytes(b)
        h = C.c_void_p()
        if lib.jl_gguf_open(str(path).encode(), C.byref(h)) != 0:
            assert lib.jl_last_error() and not h.value
            continue
        opened += 1
        count = lib.jl_gguf_tensor_count(h)
        assert count >= 0 and lib.jl_gguf_metadata_count(h) >= 0 and lib.jl_gguf_data_offset(h) >= 0
        for i in range(-1, count + 1):
            name, typ, nd = C.c_char_p(), C.c_int(), C.c_int()
            dims, off, nbytes = (C.c_int64 * 4)(), C.c_int64(), C.c_int64()
            st = lib.jl_gguf_tensor_info(h, i, C.byref(name), C.byref(typ), C.byref(nd), dims, C.byref(off), C.byref(nbytes))
            assert (st == 0) == (0 <= i < count)
            if st == 0:
                w = C.c_void_p()
                assert lib.jl_gguf_upload(None, h, name.value, C.byref(w)) != 0 and not w.value
        for key in keys:
            v, d, s, ln, et, cnt = C.c_int64(), C.c_double(), C.c_char_p(), C.c_int64(), C.c_int(), C.c_int64()
            lib.jl_gguf_metadata_int(h, key, C.byref(v))
            lib.jl_gguf_metadata_float(h, key, C.byref(d))
            if lib.jl_gguf_metadata_string(h, key, C.byref(s), C.byref(ln)) == 0:
                assert len(s.value) <= ln.value <= len(b)
            if lib.jl_gguf_metadata_array(h, key, C.byref(et), C.byref(cnt)) == 0:
                assert 0 <= cnt.value or et.value >= 0
        assert lib.jl_gguf_close(h) == 0
    assert 100 < opened < 1500
