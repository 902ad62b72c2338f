"""No-GPU checks of the boundary: the library loads, exports what include/jitllm_hip.h declares,
and its argument checks answer without a device."""
import ctypes as C
import os
import re

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def lib():
    from jitllm_amd import _lib as L
    if not os.path.exists(L.LIB):
        from jitllm_amd.build import build
        build(force=False)
    return L.load()


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "jitllm_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(jl_[a-z0-9_]+)\s*\(", text)))


def test_every_declared_symbol_is_exported_and_bound(lib):
    from jitllm_amd import _lib as L
    declared = declared_symbols()
    assert len(declared) >= 20
    for name in declared:
        assert hasattr(lib, name), f"{name} declared in jitllm_hip.h but not exported"
    assert sorted(L.SYMBOLS) == declared


def test_abi_version(lib):
    from jitllm_amd import _lib as L
    assert lib.jl_abi_version() == L.ABI_VERSION


def test_argument_checks_need_no_device(lib):
    from jitllm_amd import _lib as L
    assert lib.jl_sync(None) == L.JL_ERR_INVALID
    assert b"context is null" in lib.jl_last_error()
    assert lib.jl_gemv(None, None, None, None, 0) == L.JL_ERR_INVALID
    assert lib.jl_gemm_workspace_bytes(0, 2048, 2048, 0) == 0
    f16 = lib.jl_gemm_workspace_bytes(512, 2048, 0, L.JL_MATH_F16)
    assert f16 >= 512 * 2048 * 2 + 512 * 4 and f16 % 256 == 0
    assert lib.jl_gemm_workspace_bytes(100, 2048, 0, L.JL_MATH_F16) >= 128 * 2048 * 2
    # split-K planes grow with the output width, never beyond about twice the weight bytes
    wide = lib.jl_gemm_workspace_bytes(64, 4096, 12288, L.JL_MATH_F16)
    assert f16 < wide <= 256 * 4096 * 2 + 2048 + 12288 * 4096 * 17 // 8 + (1 << 17)
    # a thousand rows or more: room for the fp16 copy of the widest call's weights
    many = lib.jl_gemm_workspace_bytes(2048, 2048, 16384, L.JL_MATH_F16)
    assert many >= 2048 * 2048 * 2 + 16384 * 2048 * 2
    assert lib.jl_gemm_workspace_bytes(64, 4096, 12288, L.JL_MATH_DEFAULT) == wide


def test_without_a_device_context_creation_fails_loudly(lib):
    """On a box with no GPU the product path raises; it never computes on the CPU."""
    from jitllm_amd import _lib as L
    h = C.c_void_p()
    st = lib.jl_context_create(0, C.byref(h))
    if st == L.JL_OK:
        lib.jl_context_destroy(h)
        pytest.skip("a GPU is present")
    assert st in (L.JL_ERR_HIP, L.JL_ERR_INVALID, L.JL_ERR_UNSUPPORTED)
    with pytest.raises(L.JitllmHipError):
        L.check(st)


def test_package_never_imports_the_oracle():
    """The oracle is test infrastructure: nothing under jitllm_amd/ may name it."""
    pkg = os.path.join(ROOT, "jitllm_amd")
    for base, _, files in os.walk(pkg):
        for f in files:
            if f.endswith((".py", ".hip", ".h", ".cpp")):
                text = open(os.path.join(base, f), errors="replace").read()
                assert "pyoracle" not in text and "jitllm_oracle" not in text, os.path.join(base, f)
                assert not re.search(r"^\s*(from|import)\s+oracle\b", text, flags=re.M), f


def test_ggml_geometry():
    from jitllm_amd.ggml import GGMLType
    assert (GGMLType.Q8_0.block_elems, GGMLType.Q8_0.block_bytes) == (32, 34)
    assert (GGMLType.Q4_0.block_elems, GGMLType.Q4_0.block_bytes) == (32, 18)
    assert (GGMLType.Q4_K.block_elems, GGMLType.Q4_K.block_bytes) == (256, 144)
    assert GGMLType.Q8_0.byte_size_for(2048 * 2048) == 4456448
    with pytest.raises(ValueError):
        GGMLType.Q4_K.byte_size_for(100)


def test_synthetic_weights_follow_the_stated_distributions():
    from jitllm_amd import synthetic
    from jitllm_amd.ggml import GGMLType
    raw = synthetic.weight(GGMLType.Q8_0, 8, 2048, seed=3).reshape(-1, 34)
    d = raw[:, 0:2].copy().view(np.float16).astype(np.float32)
    assert d.min() >= 1e-3 * 0.999 and d.max() <= 2e-2 * 1.001
    q = raw[:, 2:].view(np.int8)
    assert q.min() == -127 and q.max() == 127
    assert np.array_equal(raw.reshape(-1), synthetic.weight(GGMLType.Q8_0, 8, 2048, seed=3))
    k = synthetic.weight(GGMLType.Q4_K, 4, 1024, seed=4)
    assert k.size == 4 * 4 * 144


def test_header_is_plain_c_and_the_library_links_from_c(lib, tmp_path):
    """The boundary is a C ABI: the header compiles as strict C99 with no other include than the
    standard ones, and a C program that knows nothing but the header links against the library and
    gets answers from the calls that need no device."""
    import shutil
    import subprocess
    from jitllm_amd import _lib as L
    gcc = shutil.which("gcc")
    if gcc is None:
        pytest.skip("no C compiler")
    src = tmp_path / "consumer.c"
    src.write_text(
        '#include "jitllm_hip.h"\n'
        '#include <stdio.h>\n'
        '#include <string.h>\n'
        'int main(void) {\n'
        '    jl_context *ctx = (jl_context *)0;\n'
        '    jl_weight *w = (jl_weight *)0;\n'
        '    unsigned char block[34] = {0};\n'
        '    int st = jl_weight_upload(ctx, JL_Q8_0, block, 1, 32, &w);\n'
        '    if (st != JL_ERR_INVALID || w != (jl_weight *)0) return 2;\n'
        '    if (strlen(jl_last_error()) == 0) return 3;\n'
        '    if (jl_gemm_workspace_bytes(64, 4096, 4096, JL_MATH_DEFAULT) == 0) return 4;\n'
        '    printf("%d\\n", jl_abi_version());\n'
        '    return 0;\n'
        '}\n')
    include = os.path.join(ROOT, "include")
    subprocess.run([gcc, "-std=c99", "-pedantic", "-Wall", "-Wextra", "-Werror", "-fsyntax-only", "-I", include, str(src)],
                   check=True)
    exe = tmp_path / "consumer"
    libdir = os.path.dirname(L.LIB)
    subprocess.run([gcc, "-std=c99", "-I", include, str(src), "-o", str(exe), "-L", libdir, "-ljitllm_hip",
                    "-Wl,-rpath," + libdir, "-Wl,-rpath,/opt/rocm/lib"], check=True)
    out = subprocess.run([str(exe)], check=True, capture_output=True, text=True).stdout
    assert int(out) == lib.jl_abi_version()
