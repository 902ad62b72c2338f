"""jl_argmax_static -- the entry point that allocates nothing -- against jl_argmax, through the C ABI.

Two calls in a row on one context, the second over a smaller input: the second call must not see
what the first left in the library's static cells.  Results are indices, so the bar is equality.
"""
import ctypes as C

import numpy as np
import pytest

from gpu_util import say
from oracle import pyoracle as O

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ctx():
    from jitllm_amd.runtime import Context
    c = Context(0)
    yield c
    c.close()


def both(ctx, values: np.ndarray):
    """(jl_argmax, jl_argmax_static) of one input, each into its own poisoned cell."""
    from jitllm_amd import _lib as L
    lib = ctx._lib
    dv = ctx.from_numpy(values)
    out = ctx.raw_buffer(8)
    out.upload(np.array([-7, -7], dtype=np.int32))
    L.check(lib.jl_argmax(ctx.handle, dv.ptr, values.size, out.ptr.value))
    L.check(lib.jl_argmax_static(ctx.handle, dv.ptr, values.size, out.ptr.value + 4))
    ctx.sync()
    a, b = out.download(np.int32, 2)
    dv.free()
    out.free()
    return int(a), int(b)


def test_static_argmax_equals_argmax_on_two_calls_the_second_smaller(ctx):
    rng = np.random.default_rng(77)
    big = rng.standard_normal(128256).astype(np.float32)
    big[100_000] = 50.0                      # far beyond the second input's length
    small = rng.standard_normal(777).astype(np.float32)
    small[5] = small[400] = 9.0               # two equal maxima: the first wins
    for name, values in (("128256 values", big), ("777 values", small)):
        say("static argmax", name)
        plain, static = both(ctx, values)
        assert plain == O.argmax(values)
        assert static == plain, name
    assert both(ctx, small)[1] == 5


@pytest.mark.parametrize("n", [1, 5, 1023, 4097])
def test_static_argmax_edges(ctx, n):
    say("static argmax edges", n)
    rng = np.random.default_rng(n)
    cases = [rng.standard_normal(n).astype(np.float32), rng.integers(0, 3, n).astype(np.float32),
             np.full(n, -np.inf, dtype=np.float32)]
    if n > 2:
        nan_first = cases[0].copy()
        nan_first[0] = np.nan
        cases.append(nan_first)
    for values in cases:
        plain, static = both(ctx, values)
        assert static == plain == O.argmax(values)


def test_static_argmax_refuses_more_than_its_maximum(ctx):
    from jitllm_amd import _lib as L
    lib = ctx._lib
    dv = ctx.float_array(4, fill=0.0)
    out = ctx.raw_buffer(4)
    st = lib.jl_argmax_static(ctx.handle, dv.ptr, (1 << 24) + 1, out.ptr)
    assert st == L.JL_ERR_INVALID
    assert b"at most" in lib.jl_last_error()
    assert lib.jl_argmax_static(ctx.handle, dv.ptr, 0, out.ptr) == L.JL_ERR_INVALID


def _hip():
    hip = C.CDLL("libamdhip64.so")
    hip.hipMemGetInfo.argtypes = [C.POINTER(C.c_size_t), C.POINTER(C.c_size_t)]
    hip.hipStreamBeginCapture.argtypes = [C.c_void_p, C.c_int]
    hip.hipStreamEndCapture.argtypes = [C.c_void_p, C.POINTER(C.c_void_p)]
    hip.hipGraphInstantiate.argtypes = [C.POINTER(C.c_void_p), C.c_void_p, C.c_void_p, C.c_void_p, C.c_size_t]
    hip.hipGraphLaunch.argtypes = [C.c_void_p, C.c_void_p]
    hip.hipGraphExecDestroy.argtypes = [C.c_void_p]
    hip.hipGraphDestroy.argtypes = [C.c_void_p]
    return hip


def _free_bytes(hip) -> int:
    free, total = C.c_size_t(), C.c_size_t()
    assert hip.hipMemGetInfo(C.byref(free), C.byref(total)) == 0
    return int(free.value)


def test_static_argmax_allocates_nothing_and_can_be_captured(ctx):
    """What the entry point is for: a burst of calls leaves the device's free memory where it was,
    and the call is legal inside a stream capture (launches only), whose replays -- with the
    program's own eager work and synchronisations between them -- give the eager index."""
    from jitllm_amd import _lib as L
    lib, hip = ctx._lib, _hip()
    say("static argmax: no allocation, capture")
    rng = np.random.default_rng(99)
    values = rng.standard_normal(50_000).astype(np.float32)
    values[31_337] = 40.0
    dv = ctx.from_numpy(values)
    other = ctx.from_numpy(rng.standard_normal(4097).astype(np.float32))
    out = ctx.raw_buffer(8)
    out.upload(np.array([-7, -7], dtype=np.int32))
    L.check(lib.jl_argmax_static(ctx.handle, dv.ptr, values.size, out.ptr.value))   # first call on the device done
    ctx.sync()
    before = _free_bytes(hip)
    for _ in range(200):
        L.check(lib.jl_argmax_static(ctx.handle, dv.ptr, values.size, out.ptr.value))
    ctx.sync()
    assert _free_bytes(hip) == before
    assert int(out.download(np.int32, 2)[0]) == 31_337
    stream = lib.jl_context_stream(ctx.handle)
    assert hip.hipStreamBeginCapture(stream, 0) == 0
    st = lib.jl_argmax_static(ctx.handle, dv.ptr, values.size, out.ptr.value)
    graph, exe = C.c_void_p(), C.c_void_p()
    assert hip.hipStreamEndCapture(stream, C.byref(graph)) == 0
    L.check(st)
    assert hip.hipGraphInstantiate(C.byref(exe), graph, None, None, 0) == 0
    hip.hipGraphDestroy(graph)
    for replay in range(4):
        out.upload(np.array([-7, -7], dtype=np.int32))
        # eager work between the replays: another input through the same static cells
        L.check(lib.jl_argmax_static(ctx.handle, other.ptr, 4097, out.ptr.value + 4))
        ctx.sync()
        assert hip.hipGraphLaunch(exe, stream) == 0
        ctx.sync()
        got = out.download(np.int32, 2)
        assert int(got[0]) == 31_337, replay
        assert int(got[1]) == O.argmax(other.get()), replay
    assert hip.hipGraphExecDestroy(exe) == 0
    # (free memory is not compared again here: instantiating a graph makes the runtime set memory
    # aside for its own bookkeeping, which is not the entry point's doing)
