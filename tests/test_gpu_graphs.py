"""Calls recorded into a HIP graph.

The reference runs its programs as captured graphs (-Djitllm.cudaGraphs); here every projection
entry point is launches only, so a warmed-up call can be recorded on the context's stream.  A
recording is only as good as its replays: each one below runs after the program's own eager work (a
new input uploaded, a synchronization) and is held bit for bit to what the same call gave eagerly
for that input -- counters that a launch leaves at zero, partial sums, decoded copies and flags that
say what a kept copy holds all have to come out the same the second and third time round.
"""
import numpy as np
import pytest

from gpu_util import say
from oracle import pyoracle as O

pytestmark = pytest.mark.gpu

UNTOUCHED = np.float32(-12345.5)


@pytest.fixture(scope="module")
def ctx():
    from jitllm_amd.runtime import Context
    c = Context(0)
    yield c
    c.close()


@pytest.fixture(scope="module")
def hip():
    import bench
    return bench.Hip()


def held_to_eager(ctx, hip, enqueue, set_input, read_output, inputs, rounds=2):
    eager = []
    for x in inputs:
        set_input(x)
        enqueue()
        ctx.sync()
        eager.append(read_output())
    assert any(not np.array_equal(eager[0], e) for e in eager[1:]), "the inputs do not tell replays apart"
    set_input(inputs[0])
    exe = hip.capture(ctx.stream, enqueue)
    try:
        for _ in range(rounds):
            for x, want in zip(inputs, eager):
                set_input(x)                      # eager work between replays: an upload and its wait
                hip.launch(exe, ctx.stream)
                ctx.sync()
                got = read_output()
                assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    finally:
        hip.destroy_graph(exe)


def test_a_decode_layer_and_the_greedy_token_replayed(ctx, hip):
    """fused q|k|v, the residual projections, gate/up + SwiGLU with the RMS scale folded in, the
    vocabulary projection that keeps its own candidates and the fold that names the token."""
    from jitllm_amd import synthetic
    from jitllm_amd.projections import QuantizedProjections, TornadoWorkspace
    say("graph: decode layer")
    t, dim, kv, ffn, vocab = O.Q8_0, 2048, 512, 8192, 32000
    w = {k: ctx.load_weight(t, synthetic.weight(t, d, n, seed=9800 + i), d, n)
         for i, (k, d, n) in enumerate([("q", dim, dim), ("k", kv, dim), ("v", kv, dim), ("o", dim, dim),
                                        ("g", ffn, dim), ("u", ffn, dim), ("d", dim, ffn), ("cls", vocab, dim)])}
    x, xb, hb = ctx.float_array(dim), ctx.float_array(dim), ctx.float_array(ffn)
    q, k, v = ctx.float_array(dim), ctx.float_array(kv), ctx.float_array(kv)
    logits, token = ctx.float_array(vocab), ctx.raw_buffer(4)
    rw = ctx.from_numpy((1.0 + 0.1 * synthetic.activations(dim, 9810)).astype(np.float32))
    proj = QuantizedProjections(ctx, TornadoWorkspace(wrapX=x, wrapXb=xb, wrapHb=hb))

    def layer():
        proj.fusedRmsNormQKV(x, q, k, v, rw, None, w["q"], w["k"], w["v"], eps=1e-5)
        proj.residualMatvec(q, w["o"], dim, dim)
        proj.fullyFusedRmsNormGateUp(x, rw, 1e-5, w["g"], w["u"], dim, ffn)
        proj.residualMatvec(hb, w["d"], ffn, dim)
        proj.matvecArgmax(x, logits, w["cls"], dim, vocab, token, rmsWeights=rw, eps=1e-5)

    inputs = [synthetic.activations(dim, 9820 + i) for i in range(3)]
    held_to_eager(ctx, hip, layer, x.set,
                  lambda: np.concatenate([x.get(), logits.get(), token.download(np.int32, 1).astype(np.float32)]), inputs)
    for t_ in w.values():
        t_.free()


@pytest.mark.parametrize("t,rows", [(O.Q4_K, 8), (O.Q4_K, 32), (O.Q8_0, 64), (O.Q6_K, 40), (O.Q4_K, 200)])
def test_batched_decode_replayed(ctx, hip, t, rows):
    """The weight-streaming kernel: its spans are folded inside the launch over counters that every
    call must leave at zero for the next -- also the next replay."""
    from jitllm_amd import synthetic
    from jitllm_amd.projections import QuantizedBatchProjections
    say("graph: batched decode", t, rows)
    dim, ffn = 2048, 4096
    wo = ctx.load_weight(t, synthetic.weight(t, dim, dim, seed=9830), dim, dim)
    w1 = ctx.load_weight(t, synthetic.weight(t, ffn, dim, seed=9831), ffn, dim)
    w3 = ctx.load_weight(t, synthetic.weight(t, ffn, dim, seed=9832), ffn, dim)
    w2 = ctx.load_weight(t, synthetic.weight(t, dim, ffn, seed=9833), dim, ffn)
    proj = QuantizedBatchProjections(ctx, rows, ffn, 2 * ffn)
    X, res, hb = ctx.float_array(rows * dim), ctx.float_array(rows * dim), ctx.float_array(rows * ffn)
    base = synthetic.activations(rows * dim, 9834)

    def calls():
        proj.projection(X, res, wo, dim, dim, True)
        proj.gateUp(X, hb, w1, w3, dim, ffn)
        proj.projection(hb, res, w2, ffn, dim, True)

    def set_input(x):
        X.set(x)
        res.set(base)          # the residual the calls add to starts over

    inputs = [synthetic.activations(rows * dim, 9840 + i) for i in range(3)]
    held_to_eager(ctx, hip, calls, set_input, lambda: np.concatenate([res.get(), hb.get()]), inputs)
    for w in (wo, w1, w3, w2):
        w.free()
    proj.workspace.free()


@pytest.mark.parametrize("mode", ["default", "resident", "xf16", "int8"])
def test_prefill_calls_replayed(ctx, hip, mode):
    """512 rows: K cut into runs with the fold launch behind them, the decode pass, a kept copy whose
    flag says what it holds (set by the first eager call, read by every replay), fp16 activations with
    an fp16 hidden vector, and the block-scaled int8 arithmetic."""
    from jitllm_amd import _lib as L, synthetic
    from jitllm_amd.projections import QuantizedBatchProjections
    say("graph: prefill", mode)
    t, rows, dim, ffn = O.Q8_0, 512, 2048, 4096
    wo = ctx.load_weight(t, synthetic.weight(t, dim, dim, seed=9850), dim, dim)
    w1 = ctx.load_weight(t, synthetic.weight(t, ffn, dim, seed=9851), ffn, dim)
    w3 = ctx.load_weight(t, synthetic.weight(t, ffn, dim, seed=9852), ffn, dim)
    w2 = ctx.load_weight(t, synthetic.weight(t, dim, ffn, seed=9853), dim, ffn)
    proj = QuantizedBatchProjections(ctx, rows, ffn, 2 * ffn, resident=mode in ("resident", "xf16"),
                                     math=L.JL_MATH_INT8 if mode == "int8" else L.JL_MATH_DEFAULT)
    res = ctx.float_array(rows * dim)
    base = synthetic.activations(rows * dim, 9854)
    if mode == "xf16":
        X, hb = ctx.half_array(rows * dim), ctx.half_array(rows * ffn)
        read = lambda: np.concatenate([res.get(), hb.get().astype(np.float32)])   # noqa: E731
    else:
        X, hb = ctx.float_array(rows * dim), ctx.float_array(rows * ffn)
        read = lambda: np.concatenate([res.get(), hb.get()])                       # noqa: E731

    def calls():
        proj.projection(X, res, wo, dim, dim, True)
        proj.gateUp(X, hb, w1, w3, dim, ffn)
        proj.projection(hb, res, w2, ffn, dim, True)

    def set_input(x):
        X.set(x.astype(np.float16) if mode == "xf16" else x)
        res.set(base)

    inputs = [synthetic.activations(rows * dim, 9860 + i) for i in range(3)]
    held_to_eager(ctx, hip, calls, set_input, read, inputs)
    for w in (wo, w1, w3, w2):
        w.free()
    proj.workspace.free()


# ---- streams and device memory that belong to the caller -------------------------------------------

def test_context_on_a_stream_the_caller_owns():
    """jl_context_create_on_stream: the calls are enqueued on the caller's stream (an event the caller
    records there after the call covers them), jl_context_stream hands the same handle back, and
    destroying the context leaves the stream alive."""
    import ctypes as C

    from jitllm_amd import synthetic
    from jitllm_amd.projections import QuantizedProjections, TornadoWorkspace
    from jitllm_amd.runtime import Context
    say("a context on the caller's stream")
    rt = C.CDLL("libamdhip64.so")
    rt.hipStreamCreate.argtypes = [C.POINTER(C.c_void_p)]
    rt.hipStreamSynchronize.argtypes = [C.c_void_p]
    rt.hipStreamDestroy.argtypes = [C.c_void_p]
    rt.hipEventCreate.argtypes = [C.POINTER(C.c_void_p)]
    rt.hipEventRecord.argtypes = [C.c_void_p, C.c_void_p]
    rt.hipEventSynchronize.argtypes = [C.c_void_p]
    rt.hipEventDestroy.argtypes = [C.c_void_p]
    stream, done = C.c_void_p(), C.c_void_p()
    assert rt.hipStreamCreate(C.byref(stream)) == 0 and rt.hipEventCreate(C.byref(done)) == 0
    t, d, n = O.Q8_0, 4096, 2048
    raw = synthetic.weight(t, d, n, seed=9870)
    x = synthetic.activations(n, seed=9871)
    c = Context(0, stream=stream.value)
    assert c.stream == stream.value
    w = c.load_weight(t, raw, d, n)
    out = c.float_array(d, fill=UNTOUCHED)
    QuantizedProjections(c, TornadoWorkspace()).floatMatvec(c.from_numpy(x), out, w, n, d)
    assert rt.hipEventRecord(done, stream) == 0 and rt.hipEventSynchronize(done) == 0
    got = out.get()
    ref = O.matmul(t, raw, x, d, n, O.DOT_VEC256)
    assert np.max(np.abs(got - ref)) <= 2e-5 * np.max(np.abs(ref)) * 50
    assert np.all(got != UNTOUCHED)
    w.free()
    c.close()
    assert rt.hipStreamSynchronize(stream) == 0      # still the caller's to use
    assert rt.hipEventDestroy(done) == 0 and rt.hipStreamDestroy(stream) == 0
