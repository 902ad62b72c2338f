"""GPU parity of the block-scaled int8 prefill GEMM (jl_gemm with JL_MATH_INT8).

The arithmetic of this path is fixed (Int8GemmKernels.java:17-23): activations quantised per
32-block to int8, each block's dot product exact in int32, acc = fma((float) dot * dA, dW, acc) over
the blocks in k order.  The kernel follows it step by step and never cuts K, so its results are held
to the oracle's statement of the same arithmetic (jo_quantize_q8 + jo_gemm_int8_block_scaled, pinned
in test_oracle_pins.py against the reference's own check) **bit for bit**.  Against the fp32 CPU path the mode is looser
by construction -- an activation carries 7 bits -- and is an opt-in like the packed decode mode: the
worst error is 2e-3 of sum |w x| on rows of 320 columns, 6e-3 on rows of 64 (fewer terms to average
over), and inside the 1e-3 bound at model row lengths.  The tests hold every output to what the
quantiser guarantees -- an activation moves by at most half a step, so |out - cpu| <= sum over the
blocks of (dA / 2) * sum |w| -- and the whole result to a relative L2 error of 2e-2 (the reference's
envelope for its integer-activation modes is 5e-2, CpuGpuParity.Q8_0_PACKED_ACTIVATION).
"""
import numpy as np
import pytest

from gpu_util import magnitude, rel_err, say
from oracle import pyoracle as O

pytestmark = pytest.mark.gpu

UNTOUCHED = np.float32(-12345.5)
BLOCK = {O.Q8_0: 34, O.Q4_0: 18}


@pytest.fixture(scope="module")
def ctx():
    from jitllm_amd.runtime import Context
    c = Context(0)
    yield c
    c.close()


def int8_reference(t, raw, X, d, n, rows=None):
    """The oracle's int8 path on (a sample of) the weight's rows: [B x rows]."""
    if rows is not None:
        raw = np.ascontiguousarray(raw.reshape(d, n // 32 * BLOCK[t])[rows]).reshape(-1)
        d = rows.size
    aq, ascale = O.quantize_q8(X)
    return O.gemm_int8_block_scaled(t, aq, ascale, raw, d)


def bits(a):
    return np.ascontiguousarray(a, dtype=np.float32).view(np.uint32)


# (type, weight rows, row length, batch, active rows): ragged shapes on the one-wave tile, the
# reference's own check shape (m = 256, n = 384, k = 320), and shapes wide enough for the 128 x 128 tile
SHAPES = [
    (O.Q8_0, 200, 320, 70, 70),
    (O.Q4_0, 200, 320, 70, 70),
    (O.Q8_0, 384, 320, 256, 256),
    (O.Q4_0, 384, 320, 256, 256),
    (O.Q8_0, 37, 512, 9, 5),
    (O.Q4_0, 37, 512, 16, 16),
    (O.Q8_0, 130, 64, 130, 129),
]


@pytest.mark.parametrize("t,d,n,batch,rows", SHAPES)
@pytest.mark.parametrize("residual", [False, True])
def test_int8_projection_equals_the_oracle_bit_for_bit(ctx, t, d, n, batch, rows, residual):
    from jitllm_amd import _lib as L, synthetic
    from jitllm_amd.projections import QuantizedBatchProjections
    say("int8 projection", t, d, n, batch, rows, residual)
    raw = synthetic.weight(t, d, n, seed=2100 + d)
    X = synthetic.activations((batch, n), seed=2101)
    X[0, :32] = 0.0                      # an all-zero block: scale 0, quants 0
    X[min(3, batch - 1), 32:64] *= 1e-30  # a tiny block
    if n >= 128:
        X[min(5, batch - 1), 96:128] *= 1e-38   # below RECIPROCAL_FINITE_AMAX: the (x / amax) * 127 form, subnormal scale
    start = synthetic.activations((batch, d), seed=2102) if residual else np.full((batch, d), UNTOUCHED, np.float32)
    w = ctx.load_weight(t, raw, d, n)
    proj = QuantizedBatchProjections(ctx, batch, n, d, math=L.JL_MATH_INT8)
    out = ctx.from_numpy(start)
    proj.projection(ctx.from_numpy(X), out, w, n, d, residual, activeRows=rows)
    ctx.sync()
    got = out.get().reshape(batch, d)
    ref = int8_reference(t, raw, X[:rows], d, n)
    want = (start[:rows] + ref) if residual else ref
    assert np.array_equal(bits(got[:rows]), bits(want))
    assert np.array_equal(bits(got[rows:]), bits(start[rows:]))
    # and the fp32 CPU path, to the looser envelope of an integer-activation mode
    cpu = O.matmul_batch(t, raw, X[:rows], d, n, O.DOT_VEC256).astype(np.float64) + (start[:rows] if residual else 0.0)
    _, ascale = O.quantize_q8(X[:rows])
    wabs = np.abs(O.dequant(t, raw).reshape(d, n // 32, 32).astype(np.float64)).sum(axis=2)
    half_step = (ascale.astype(np.float64) / 2) @ wabs.T
    slack = 1e-5 * magnitude(t, raw, X[:rows], d, n) + np.abs(start[:rows]) * 1e-6 * residual
    assert np.all(np.abs(got[:rows] - cpu) <= half_step * 1.001 + slack)
    assert np.linalg.norm(got[:rows] - cpu) / np.linalg.norm(cpu) < 2e-2
    w.free()


@pytest.mark.parametrize("t", [O.Q8_0, O.Q4_0])
def test_int8_fused_qkv_side_by_side(ctx, t):
    """Three weights of ragged row counts in one call: C = X . [Wq | Wk | Wv]^T."""
    from jitllm_amd import _lib as L, synthetic
    from jitllm_amd.projections import QuantizedBatchProjections
    say("int8 qkv", t)
    n, T, ds = 256, 100, (200, 72, 65)
    raws = [synthetic.weight(t, d, n, seed=2110 + i) for i, d in enumerate(ds)]
    ws = [ctx.load_weight(t, r, d, n) for r, d in zip(raws, ds)]
    X = synthetic.activations((T, n), seed=2113)
    out = ctx.float_array(T * sum(ds), fill=UNTOUCHED)
    QuantizedBatchProjections(ctx, T, n, sum(ds), math=L.JL_MATH_INT8).fusedQKV(ctx.from_numpy(X), out, *ws)
    ctx.sync()
    got = out.get().reshape(T, sum(ds))
    want = np.concatenate([int8_reference(t, r, X, d, n) for r, d in zip(raws, ds)], axis=1)
    assert np.array_equal(bits(got), bits(want))


@pytest.mark.parametrize("t,d,n,T", [(O.Q8_0, 200, 256, 70), (O.Q4_0, 8192, 2048, 512)])
def test_int8_gate_up_swiglu(ctx, t, d, n, T):
    """SiLU(gate) * up of two int8 projections; the second shape takes the 128 x 128 tile."""
    from jitllm_amd import _lib as L, synthetic
    from jitllm_amd.projections import QuantizedBatchProjections
    say("int8 gate/up", t, d, n, T)
    r1, r3 = synthetic.weight(t, d, n, seed=2120), synthetic.weight(t, d, n, seed=2121)
    w1, w3 = ctx.load_weight(t, r1, d, n), ctx.load_weight(t, r3, d, n)
    X = synthetic.activations((T, n), seed=2122)
    hb = ctx.float_array(T * d, fill=UNTOUCHED)
    QuantizedBatchProjections(ctx, T, n, 2 * d, math=L.JL_MATH_INT8).gateUp(ctx.from_numpy(X), hb, w1, w3, n, d)
    ctx.sync()
    got = hb.get().reshape(T, d)
    assert np.all(got != UNTOUCHED)
    rows = np.unique(np.concatenate([np.arange(min(40, d)), np.arange(d - min(40, d), d),
                                     np.random.default_rng(5).choice(d, size=min(d, 64), replace=False)]))
    g = int8_reference(t, r1, X, d, n, rows).astype(np.float64)
    u = int8_reference(t, r3, X, d, n, rows).astype(np.float64)
    want = g / (1.0 + np.exp(-g)) * u
    assert np.max(np.abs(got[:, rows] - want) / (np.abs(want) + 1e-6 * np.abs(u) + 1e-30)) < 1e-5
    w1.free()
    w3.free()


@pytest.mark.parametrize("t,d,n,T", [(O.Q8_0, 8192, 2048, 768), (O.Q8_0, 2048, 8192, 512), (O.Q4_0, 3072, 2048, 2048)])
def test_int8_prefill_shapes_on_a_sample(ctx, t, d, n, T):
    """Llama-3.2-1B prefill shapes (gate-sized on the 128 x 128 tile, the down projection's 8192
    columns, q|k|v-sized at 2048 tokens): the whole call on the GPU, a sample of weight rows
    against the oracle, bit for bit."""
    from jitllm_amd import _lib as L, synthetic
    from jitllm_amd.projections import QuantizedBatchProjections
    say("int8 prefill shape", t, d, n, T)
    raw = synthetic.weight(t, d, n, seed=2130 + d % 13)
    w = ctx.load_weight(t, raw, d, n)
    X = synthetic.activations((T, n), seed=2131)
    out = ctx.float_array(T * d, fill=UNTOUCHED)
    QuantizedBatchProjections(ctx, T, n, d, math=L.JL_MATH_INT8).projection(ctx.from_numpy(X), out, w, n, d, False)
    ctx.sync()
    got = out.get().reshape(T, d)
    assert np.all(got != UNTOUCHED)
    rng = np.random.default_rng(2132)
    rows = np.unique(np.concatenate([np.arange(16), np.arange(d - 16, d), rng.choice(d, size=96, replace=False)]))
    arows = np.unique(np.concatenate([np.arange(8), np.arange(T - 8, T), rng.choice(T, size=48, replace=False)]))
    ref = int8_reference(t, raw, X[arows], d, n, rows)
    assert np.array_equal(bits(got[np.ix_(arows, rows)]), bits(ref))
    w.free()


def _sample(count, total, seed):
    rng = np.random.default_rng(seed)
    return np.unique(np.concatenate([np.arange(min(16, total)), np.arange(max(0, total - 16), total),
                                     rng.choice(total, size=min(count, total), replace=False)]))


def test_int8_big_tile_gate_up_q8_0_with_ragged_rows(ctx):
    """Q8_0 gate/up on the 128 x 128 tile (4100 weight rows: the last tile of each weight is ragged,
    1000 of 1024 activation rows active)."""
    from jitllm_amd import _lib as L, synthetic
    from jitllm_amd.projections import QuantizedBatchProjections
    t, d, n, T, active = O.Q8_0, 4100, 1024, 1024, 1000
    say("int8 big-tile gate/up", d, n, T)
    r1, r3 = synthetic.weight(t, d, n, seed=2150), synthetic.weight(t, d, n, seed=2151)
    w1, w3 = ctx.load_weight(t, r1, d, n), ctx.load_weight(t, r3, d, n)
    X = synthetic.activations((T, n), seed=2152)
    hb = ctx.float_array(T * d, fill=UNTOUCHED)
    QuantizedBatchProjections(ctx, T, n, 2 * d, math=L.JL_MATH_INT8).gateUp(ctx.from_numpy(X), hb, w1, w3, n, d,
                                                                            activeRows=active)
    ctx.sync()
    got = hb.get().reshape(T, d)
    assert np.all(got[:active] != UNTOUCHED) and np.all(got[active:] == UNTOUCHED)
    rows, arows = _sample(64, d, 2153), _sample(32, active, 2154)
    g = int8_reference(t, r1, X[arows], d, n, rows).astype(np.float64)
    u = int8_reference(t, r3, X[arows], d, n, rows).astype(np.float64)
    want = g / (1.0 + np.exp(-g)) * u
    assert np.max(np.abs(got[np.ix_(arows, rows)] - want) / (np.abs(want) + 1e-6 * np.abs(u) + 1e-30)) < 1e-5
    w1.free()
    w3.free()


def test_int8_big_tile_residual_with_ragged_rows(ctx):
    """JL_RESIDUAL through the 128 x 128 tile: 3100 weight rows (a ragged last tile), 2048 tokens."""
    from jitllm_amd import _lib as L, synthetic
    from jitllm_amd.projections import QuantizedBatchProjections
    t, d, n, T = O.Q8_0, 3100, 1024, 2048
    say("int8 big-tile residual", d, n, T)
    raw = synthetic.weight(t, d, n, seed=2160)
    w = ctx.load_weight(t, raw, d, n)
    X = synthetic.activations((T, n), seed=2161)
    start = synthetic.activations((T, d), seed=2162)
    out = ctx.from_numpy(start)
    QuantizedBatchProjections(ctx, T, n, d, math=L.JL_MATH_INT8).projection(ctx.from_numpy(X), out, w, n, d, True)
    ctx.sync()
    got = out.get().reshape(T, d)
    rows, arows = _sample(96, d, 2163), _sample(48, T, 2164)
    ref = int8_reference(t, raw, X[arows], d, n, rows)
    assert np.array_equal(bits(got[np.ix_(arows, rows)]), bits(start[np.ix_(arows, rows)] + ref))
    w.free()


@pytest.mark.parametrize("t", [O.Q8_0, O.Q4_0])
def test_int8_big_tile_three_weights_side_by_side(ctx, t):
    """q|k|v of 2048, 520 and 520 rows at 2048 tokens: three weights, each with a ragged last tile,
    on the 128 x 128 tile (where a weight's first tile and first output column are looked up)."""
    from jitllm_amd import _lib as L, synthetic
    from jitllm_amd.projections import QuantizedBatchProjections
    n, T, ds = 1024, 2048, (2048, 520, 520)
    say("int8 big-tile q|k|v", t)
    raws = [synthetic.weight(t, d, n, seed=2170 + i) for i, d in enumerate(ds)]
    ws = [ctx.load_weight(t, r, d, n) for r, d in zip(raws, ds)]
    X = synthetic.activations((T, n), seed=2173)
    out = ctx.float_array(T * sum(ds), fill=UNTOUCHED)
    QuantizedBatchProjections(ctx, T, n, sum(ds), math=L.JL_MATH_INT8).fusedQKV(ctx.from_numpy(X), out, *ws)
    ctx.sync()
    got = out.get().reshape(T, sum(ds))
    assert np.all(got != UNTOUCHED)
    arows = _sample(32, T, 2174)
    col = 0
    for raw, d in zip(raws, ds):
        rows = _sample(48, d, 2175 + d)
        ref = int8_reference(t, raw, X[arows], d, n, rows)
        assert np.array_equal(bits(got[np.ix_(arows, col + rows)]), bits(ref))
        col += d
    for w in ws:
        w.free()


def test_int8_refusals(ctx):
    import ctypes as C
    from jitllm_amd import _lib as L, synthetic
    say("int8 refusals")
    lib = L.load()
    w = ctx.load_weight(O.Q8_0, synthetic.weight(O.Q8_0, 64, 96, 1), 64, 96)    # 96 columns: not whole pairs
    x, o = ctx.float_array(4 * 96, 0.0), ctx.float_array(4 * 64, 0.0)
    arr = (C.c_void_p * 1)(w.handle)
    ws = ctx.raw_buffer(1 << 20)
    st = lib.jl_gemm(ctx.handle, arr, 1, x.ptr, o.ptr, 4, 4, 64, 0, L.JL_STORE, L.JL_MATH_INT8, ws.ptr, ws.nbytes)
    assert st == L.JL_ERR_UNSUPPORTED and b"multiple of 64" in lib.jl_last_error()
    w2 = ctx.load_weight(O.Q8_0, synthetic.weight(O.Q8_0, 64, 128, 1), 64, 128)
    arr2 = (C.c_void_p * 1)(w2.handle)
    st = lib.jl_gemm(ctx.handle, arr2, 1, x.ptr, o.ptr, 3, 3, 64, 0, L.JL_STORE, L.JL_MATH_INT8, ws.ptr, 256)
    assert st == L.JL_ERR_WORKSPACE
    w6 = ctx.load_weight(O.Q6_K, synthetic.weight(O.Q6_K, 64, 256, 1), 64, 256)
    arr6 = (C.c_void_p * 1)(w6.handle)
    st = lib.jl_gemm(ctx.handle, arr6, 1, x.ptr, o.ptr, 1, 1, 64, 0, L.JL_STORE, L.JL_MATH_INT8, ws.ptr, ws.nbytes)
    assert st == L.JL_ERR_UNSUPPORTED and b"Q6_K" in lib.jl_last_error()


def test_int8_row_stride_and_column_offset(ctx):
    """Two calls fill one packed row side by side (ldo, col_offset: gemmInt8Q8_0's contract,
    Int8GemmKernels.java:651-676); what lies between and beside them is left alone."""
    import ctypes as C
    from jitllm_amd import _lib as L, synthetic
    say("int8 ldo / col_offset")
    lib = L.load()
    t, n, T, da, db, ldo = O.Q8_0, 192, 37, 70, 40, 128
    ra, rb = synthetic.weight(t, da, n, seed=2140), synthetic.weight(t, db, n, seed=2141)
    wa, wb = ctx.load_weight(t, ra, da, n), ctx.load_weight(t, rb, db, n)
    X = synthetic.activations((T, n), seed=2142)
    out = ctx.float_array(T * ldo, fill=UNTOUCHED)
    nbytes = lib.jl_gemm_workspace_bytes(T, n, da, L.JL_MATH_INT8)
    ws = ctx.raw_buffer(nbytes)
    xd = ctx.from_numpy(X)
    for w, off in ((wa, 4), (wb, 80)):
        arr = (C.c_void_p * 1)(w.handle)
        L.check(lib.jl_gemm(ctx.handle, arr, 1, xd.ptr, out.ptr, T, T, ldo, off, L.JL_STORE, L.JL_MATH_INT8,
                            ws.ptr, ws.nbytes))
    ctx.sync()
    got = out.get().reshape(T, ldo)
    assert np.array_equal(bits(got[:, 4:4 + da]), bits(int8_reference(t, ra, X, da, n)))
    assert np.array_equal(bits(got[:, 80:80 + db]), bits(int8_reference(t, rb, X, db, n)))
    mask = np.ones(ldo, dtype=bool)
    mask[4:4 + da] = False
    mask[80:80 + db] = False
    assert np.all(got[:, mask] == UNTOUCHED)
