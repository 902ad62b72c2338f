"""GPU parity: batched decode and batched prefill (jl_gemm) through the C ABI."""
import numpy as np
import pytest

import fixtures as FX
from gpu_util import magnitude, rel_err, say
from oracle import pyoracle as O

pytestmark = pytest.mark.gpu

NAMES = {O.Q8_0: "q8_0", O.Q4_0: "q4_0", O.Q4_K: "q4_K"}
UNTOUCHED = np.float32(-12345.5)  # BatchProjectionTilingAccelTest.java:61
F16_BOUND = 2e-3                  # fp16-MFMA path: max |d| / sum |w x|


@pytest.fixture(scope="module")
def ctx():
    from jitllm_amd.runtime import Context
    c = Context(0)
    yield c
    c.close()


@pytest.mark.parametrize("t,what", [(O.Q4_0, "q40"), (O.Q4_K, "q4k"), (O.Q8_0, "q80")])
def test_batch_projection_reference_fixture(ctx, t, what):
    """BatchProjectionTilingAccelTest.java:151-215: N = 512, D = 37, widths {1,2,7,8,9,16},
    activeRows in {1, width}; plain and residual; rows past activeRows keep -12345.5 exactly."""
    from jitllm_amd.projections import QuantizedBatchProjections
    raw = FX.probe_blocks(t, 20260909 + O.java_string_hash(what), both_scales=(t == O.Q4_K))
    w = ctx.load_weight(t, raw, FX.D_PROBE, FX.N_PROBE)
    for width in (1, 2, 7, 8, 9, 16):
        for active in ([1] if width == 1 else [1, width]):
            say("batch fixture", what, width, active)
            X = FX.batch_activation(width)
            expected = O.matmul_batch(t, raw, X[:active], FX.D_PROBE, FX.N_PROBE)
            mag = magnitude(t, raw, X[:active], FX.D_PROBE, FX.N_PROBE)
            proj = QuantizedBatchProjections(ctx, width, FX.N_PROBE, FX.D_PROBE)
            xd = ctx.from_numpy(X)
            for residual in (False, True):
                out = ctx.float_array(width * FX.D_PROBE, fill=UNTOUCHED)
                proj.projection(xd, out, w, FX.N_PROBE, FX.D_PROBE, residual, activeRows=active)
                ctx.sync()
                got = out.get().reshape(width, FX.D_PROBE)
                assert np.all(got[active:] == UNTOUCHED)
                want = expected + (UNTOUCHED if residual else np.float32(0))
                assert rel_err(got[:active], want, mag + (12345.5 * 6e-8 if residual else 0)) < F16_BOUND


@pytest.mark.parametrize("t,d,n,B", [
    (O.Q4_K, 4096, 4096, 8), (O.Q4_K, 1024, 4096, 32), (O.Q4_K, 4096, 12288, 64),
    (O.Q8_0, 2048, 2048, 64), (O.Q4_0, 1024, 4096, 33), (O.Q8_0, 200, 2048, 130),
])
def test_batched_projection_matches_oracle(ctx, t, d, n, B):
    from jitllm_amd import synthetic
    from jitllm_amd.projections import QuantizedBatchProjections
    say("batched", NAMES[t], d, n, B)
    raw = synthetic.weight(t, d, n, seed=7000 + d)
    X = synthetic.activations((B, n), seed=7100 + B)
    ref = O.matmul_batch(t, raw, X, d, n, O.DOT_SCALAR if t == O.Q4_K else O.DOT_VEC256)
    w = ctx.load_weight(t, raw, d, n)
    out = ctx.float_array(B * d, fill=UNTOUCHED)
    QuantizedBatchProjections(ctx, B, n, d).projection(ctx.from_numpy(X), out, w, n, d, False)
    ctx.sync()
    got = out.get().reshape(B, d)
    assert np.all(got != UNTOUCHED)
    err = rel_err(got, ref, magnitude(t, raw, X, d, n))
    assert err < F16_BOUND, err
    assert err < 2e-4, err  # random rounding errors: far inside the worst-case bound


@pytest.mark.parametrize("t", [O.Q8_0, O.Q4_0, O.Q4_K])
@pytest.mark.parametrize("d,n,rows", [(512, 4096, 8), (200, 2304, 5), (96, 12288, 1)])
def test_calls_of_at_most_eight_rows_match_the_same_rows_of_a_larger_call(ctx, t, d, n, rows):
    """Calls of at most 8 rows run an instance of the weight-streaming kernel whose prologue skips
    rows 8..15 of the row block.  A row's scale, fragments and sums do not depend on the other rows
    (FloatTensor.java:127-140: row b is a dot of its own), so the results must equal the first rows
    of a 12-row call over the same activations bit for bit -- plain, residual and gate/up -- and
    meet the oracle."""
    from jitllm_amd import synthetic
    from jitllm_amd.projections import QuantizedBatchProjections
    say("at most eight rows", NAMES[t], d, n, rows)
    raw = synthetic.weight(t, d, n, seed=7300 + d)
    raw_up = synthetic.weight(t, d, n, seed=7301 + d)
    X = synthetic.activations((12, n), seed=7302 + rows)
    w, w_up = ctx.load_weight(t, raw, d, n), ctx.load_weight(t, raw_up, d, n)
    big = QuantizedBatchProjections(ctx, 12, n, 2 * d)
    small = QuantizedBatchProjections(ctx, rows, n, 2 * d)
    xd, xs = ctx.from_numpy(X), ctx.from_numpy(X[:rows])
    results = []
    for proj, x, b in ((big, xd, 12), (small, xs, rows)):
        plain, res, hb = ctx.float_array(b * d), ctx.float_array(b * d, fill=1.5), ctx.float_array(b * d)
        proj.projection(x, plain, w, n, d, False)
        proj.projection(x, res, w, n, d, True)
        proj.gateUp(x, hb, w, w_up, n, d)
        ctx.sync()
        results.append([a.get().reshape(b, d)[:rows] for a in (plain, res, hb)])
    for a, b in zip(*results):
        assert np.array_equal(a, b)
    ref = O.matmul_batch(t, raw, X[:rows], d, n, O.DOT_SCALAR if t == O.Q4_K else O.DOT_VEC256)
    assert rel_err(results[1][0], ref, magnitude(t, raw, X[:rows], d, n)) < 2e-4


def _random_batched_shapes():
    """Seeded shapes across the weight-streaming kernel's launch geometries: one to eight compute
    waves per workgroup (row lengths of 256 .. 2048 columns per span), one, two and several spans
    per row, one or two row blocks per workgroup, two row blocks across the grid, partial batches."""
    rng = np.random.default_rng(20261125)
    shapes = []
    for t in (O.Q8_0, O.Q4_0, O.Q4_K):
        for n in (256, 768, 1280, 2048, 2304, 4096, 6144):
            rows = int(rng.choice([1, 3, 8, 9, 16, 17, 31, 32, 33, 50, 64]))
            d = int(rng.integers(1, 300))
            active = rows if rng.integers(0, 2) else int(rng.integers(1, rows + 1))
            shapes.append((t, d, n, rows, active))
    return shapes


@pytest.mark.parametrize("t,d,n,rows,active", _random_batched_shapes())
def test_batched_decode_on_random_shapes(ctx, t, d, n, rows, active):
    """Plain, residual and gate/up results of the weight-streaming kernel against the oracle; rows
    past the active ones keep their contents (BatchProjectionTilingAccelTest.java:151-215)."""
    from jitllm_amd import synthetic
    from jitllm_amd.projections import QuantizedBatchProjections
    say("batched, random shape", NAMES[t], d, n, rows, active)
    raw = synthetic.weight(t, d, n, seed=7500 + d)
    raw_up = synthetic.weight(t, d, n, seed=7501 + d)
    X = synthetic.activations((rows, n), seed=7502 + n)
    dot = O.DOT_SCALAR if t == O.Q4_K else O.DOT_VEC256
    g = O.matmul_batch(t, raw, X[:active], d, n, dot)
    u = O.matmul_batch(t, raw_up, X[:active], d, n, dot)
    mg, mu = magnitude(t, raw, X[:active], d, n), magnitude(t, raw_up, X[:active], d, n)
    w, w_up = ctx.load_weight(t, raw, d, n), ctx.load_weight(t, raw_up, d, n)
    proj = QuantizedBatchProjections(ctx, rows, n, 2 * d)
    xd = ctx.from_numpy(X)
    plain = ctx.float_array(rows * d, fill=UNTOUCHED)
    res = ctx.float_array(rows * d, fill=UNTOUCHED)
    hb = ctx.float_array(rows * d, fill=UNTOUCHED)
    proj.projection(xd, plain, w, n, d, False, activeRows=active)
    proj.projection(xd, res, w, n, d, True, activeRows=active)
    proj.gateUp(xd, hb, w, w_up, n, d, activeRows=active)
    ctx.sync()
    plain, res, hb = (a.get().reshape(rows, d) for a in (plain, res, hb))
    for a in (plain, res, hb):
        assert np.all(a[active:] == UNTOUCHED)
    assert rel_err(plain[:active], g, mg) < F16_BOUND
    assert rel_err(res[:active], g + UNTOUCHED, mg + 12345.5 * 6e-8) < F16_BOUND
    ref = O.swiglu(g.reshape(-1), u.reshape(-1)).reshape(active, d)
    bound = F16_BOUND * (mg * np.abs(u) + 1.2 * mu * np.abs(g)) + 1e-6
    assert np.all(np.abs(hb[:active].astype(np.float64) - ref) <= bound)


def test_batched_row_is_the_single_vector_result(ctx):
    """FloatTensor.java:127-140: batched row b is the same dot as the single-vector call, so the
    batched kernel's rows must agree with each other when their activations are equal."""
    from jitllm_amd import synthetic
    from jitllm_amd.projections import QuantizedBatchProjections
    say("batched equal rows")
    d, n, B = 512, 2048, 12
    raw = synthetic.weight(O.Q8_0, d, n, seed=71)
    x = synthetic.activations(n, seed=72)
    X = np.tile(x, (B, 1))
    out = ctx.float_array(B * d)
    QuantizedBatchProjections(ctx, B, n, d).projection(ctx.from_numpy(X), out,
                                                    ctx.load_weight(O.Q8_0, raw, d, n), n, d, False)
    ctx.sync()
    got = out.get().reshape(B, d)
    assert np.all(got == got[0])


@pytest.mark.parametrize("t,dq,dkv,n,T", [(O.Q8_0, 2048, 512, 2048, 256), (O.Q4_K, 256, 128, 1024, 70)])
def test_prefill_fused_qkv_side_by_side(ctx, t, dq, dkv, n, T):
    """C = A . [Wq|Wk|Wv]^T with the outputs side by side (FP16Projections / DecodedMatMul.project)."""
    from jitllm_amd import synthetic
    from jitllm_amd.projections import QuantizedBatchProjections
    say("prefill qkv", NAMES[t], dq, dkv, n, T)
    dims = (dq, dkv, dkv)
    raws = [synthetic.weight(t, d, n, seed=81 + i) for i, d in enumerate(dims)]
    X = synthetic.activations((T, n), seed=85)
    ws = [ctx.load_weight(t, r, d, n) for r, d in zip(raws, dims)]
    ld = sum(dims)
    out = ctx.float_array(T * ld, fill=UNTOUCHED)
    QuantizedBatchProjections(ctx, T, n, ld).fusedQKV(ctx.from_numpy(X), out, *ws)
    ctx.sync()
    got = out.get().reshape(T, ld)
    col = 0
    for raw, d in zip(raws, dims):
        ref = O.matmul_batch(t, raw, X, d, n)
        assert rel_err(got[:, col:col + d], ref, magnitude(t, raw, X, d, n)) < 2e-4
        col += d


@pytest.mark.parametrize("t,d,n,T", [(O.Q8_0, 1024, 2048, 96), (O.Q4_K, 200, 512, 9), (O.Q4_0, 96, 1024, 130)])
def test_batched_gate_up(ctx, t, d, n, T):
    """hb = SiLU(w1 . x) * (w3 . x) per row (BatchProjectionTilingAccelTest.java:409, fused gate/up)."""
    from jitllm_amd import synthetic
    from jitllm_amd.projections import QuantizedBatchProjections
    say("batched gate_up", NAMES[t], d, n, T)
    r1 = synthetic.weight(t, d, n, seed=91)
    r3 = synthetic.weight(t, d, n, seed=92)
    X = synthetic.activations((T, n), seed=93)
    g = O.matmul_batch(t, r1, X, d, n)
    u = O.matmul_batch(t, r3, X, d, n)
    ref = O.swiglu(g.reshape(-1), u.reshape(-1)).reshape(T, d)
    hb = ctx.float_array(T * d, fill=UNTOUCHED)
    QuantizedBatchProjections(ctx, T, n, 2 * d).gateUp(ctx.from_numpy(X), hb, ctx.load_weight(t, r1, d, n),
                                                ctx.load_weight(t, r3, d, n), n, d)
    ctx.sync()
    got = hb.get().reshape(T, d)
    mg, mu = magnitude(t, r1, X, d, n), magnitude(t, r3, X, d, n)
    bound = 2e-4 * (mg * np.abs(u) + 1.2 * mu * np.abs(g)) + 1e-6
    assert np.all(np.abs(got.astype(np.float64) - ref) <= bound)


@pytest.mark.parametrize("t,d,n,T,residual", [
    (O.Q8_0, 300, 512, 1100, False), (O.Q8_0, 300, 512, 1100, True), (O.Q4_K, 136, 1024, 1024, False),
    (O.Q8_0, 16384, 256, 1024, False), (O.Q4_0, 2944, 4096, 1024, True),
])
def test_many_row_prefill_matches_oracle(ctx, t, d, n, T, residual):
    """A thousand rows or more: weights decoded to fp16 once per call, then the plain fp16 GEMM
    (dequantize*ToFP16 + gemmMMA, TransformerBatchPrefillKernels.java:917-1076,2325-2363).  Same
    arithmetic as the fused kernel, so the same bound; the shapes take different tiles (256 x 256,
    256 x 128, 128 x 128)."""
    from jitllm_amd import synthetic
    from jitllm_amd.projections import QuantizedBatchProjections
    say("many-row prefill", NAMES[t], d, n, T, residual)
    raw = synthetic.weight(t, d, n, seed=7300 + d)
    X = synthetic.activations((T, n), seed=7400 + T)
    ref = O.matmul_batch(t, raw, X, d, n)
    out = ctx.float_array(T * d, fill=UNTOUCHED)
    QuantizedBatchProjections(ctx, T, n, d).projection(ctx.from_numpy(X), out, ctx.load_weight(t, raw, d, n),
                                                       n, d, residual)
    ctx.sync()
    got = out.get().reshape(T, d)
    want = ref + (UNTOUCHED if residual else np.float32(0))
    err = rel_err(got, want, magnitude(t, raw, X, d, n) + (12345.5 * 6e-8 if residual else 0))
    assert err < 2e-4, err


def test_many_row_prefill_qkv_and_gate_up(ctx):
    from jitllm_amd import synthetic
    from jitllm_amd.projections import QuantizedBatchProjections
    say("many-row prefill qkv / gate_up")
    t, n, T = O.Q4_0, 512, 1024
    dims = (256, 96, 96)
    raws = [synthetic.weight(t, d, n, seed=181 + i) for i, d in enumerate(dims)]
    X = synthetic.activations((T, n), seed=185)
    ws = [ctx.load_weight(t, r, d, n) for r, d in zip(raws, dims)]
    ld = sum(dims)
    out = ctx.float_array(T * ld, fill=UNTOUCHED)
    QuantizedBatchProjections(ctx, T, n, ld).fusedQKV(ctx.from_numpy(X), out, *ws)
    ctx.sync()
    got = out.get().reshape(T, ld)
    col = 0
    for raw, d in zip(raws, dims):
        ref = O.matmul_batch(t, raw, X, d, n)
        assert rel_err(got[:, col:col + d], ref, magnitude(t, raw, X, d, n)) < 2e-4
        col += d
    # gate/up with SwiGLU; 200 outputs do not fill the last tile
    t, d, n, T = O.Q4_K, 200, 512, 1030
    r1 = synthetic.weight(t, d, n, seed=191)
    r3 = synthetic.weight(t, d, n, seed=192)
    X = synthetic.activations((T, n), seed=193)
    g = O.matmul_batch(t, r1, X, d, n)
    u = O.matmul_batch(t, r3, X, d, n)
    ref = O.swiglu(g.reshape(-1), u.reshape(-1)).reshape(T, d)
    hb = ctx.float_array(T * d, fill=UNTOUCHED)
    QuantizedBatchProjections(ctx, T, n, 2 * d).gateUp(ctx.from_numpy(X), hb, ctx.load_weight(t, r1, d, n),
                                                ctx.load_weight(t, r3, d, n), n, d)
    ctx.sync()
    got = hb.get().reshape(T, d)
    mg, mu = magnitude(t, r1, X, d, n), magnitude(t, r3, X, d, n)
    bound = 2e-4 * (mg * np.abs(u) + 1.2 * mu * np.abs(g)) + 1e-6
    assert np.all(np.abs(got.astype(np.float64) - ref) <= bound)


@pytest.mark.parametrize("t,d,n,T,residual", [
    (O.Q8_0, 5800, 256, 1024, False),    # 256 x 128 tiles, last tile 40 columns
    (O.Q4_K, 6016, 256, 1024, True),     # 256 x 128 tiles, residual
    (O.Q4_0, 12700, 256, 1100, False),   # 256 x 256 tiles (5 x 50: one round), ragged rows and columns
    (O.Q4_0, 16500, 256, 1100, False),   # 256 x 128 tiles in three rounds (5 x 65 of 256 x 256 would be two)
    (O.Q8_0, 3000, 2048, 1024, True),    # 128 x 128 tiles, K whole, last tile 56 columns
    (O.Q4_K, 3000, 1024, 600, False),    # 128 x 128 tiles, K cut in two, ragged rows
    (O.Q8_0, 1500, 2048, 512, True),     # 128 x 128 tiles, K cut in four, last tile 92 columns
    (O.Q4_0, 700, 2048, 520, False),     # 128 x 128 tiles, K cut in eight runs of four steps, ragged both ways
    (O.Q8_0, 3072, 256, 2000, False),    # 128 x 192 tiles (16 x 16 of them), ragged rows
    (O.Q4_K, 6144, 256, 2000, True),     # 256 x 192 tiles (8 x 32), ragged rows, residual
    (O.Q4_0, 3072, 512, 4096, True),     # 256 x 192 tiles (16 x 16), whole rows
])
def test_two_pass_prefill_tiles_and_edges(ctx, t, d, n, T, residual):
    """Shapes with enough tiles for the decode-once path on 256 compute units, one per tiling it
    can choose, with output columns and rows that do not fill the last tiles."""
    from jitllm_amd import synthetic
    from jitllm_amd.projections import QuantizedBatchProjections
    say("two-pass prefill", NAMES[t], d, n, T, residual)
    raw = synthetic.weight(t, d, n, seed=8300 + d)
    X = synthetic.activations((T, n), seed=8400 + T)
    ref = O.matmul_batch(t, raw, X, d, n)
    out = ctx.float_array(T * d + 64, fill=UNTOUCHED)
    QuantizedBatchProjections(ctx, T, n, d).projection(ctx.from_numpy(X), out, ctx.load_weight(t, raw, d, n),
                                                       n, d, residual)
    ctx.sync()
    flat = out.get()
    assert np.all(flat[T * d:] == UNTOUCHED)   # nothing written past the last row
    got = flat[:T * d].reshape(T, d)
    want = ref.astype(np.float64) + (float(UNTOUCHED) if residual else 0.0)
    # short rows average the fp16 rounding of the weights less: 5e-4 of sum |w x| (the path's bound
    # is 2e-3); a residual adds the rounding of the fp32 sum, half an ulp of the value it is added to
    slack = abs(np.spacing(np.float32(UNTOUCHED))) / 2 if residual else 0.0
    excess = np.abs(got.astype(np.float64) - want) - slack
    assert np.all(excess <= 5e-4 * magnitude(t, raw, X, d, n)), float(excess.max())


def _random_prefill_shapes():
    """Seeded many-row shapes across both prefill kernels and every tiling: 65 .. 1400 rows, row
    lengths of 256 .. 4096 columns, output widths from a fraction of a tile to dozens of tiles,
    partial batches, both epilogues (sizes kept to what the oracle multiplies in seconds)."""
    rng = np.random.default_rng(20261126)
    shapes = []
    for t in (O.Q8_0, O.Q4_0, O.Q4_K):
        for n in (256, 1024, 2048, 4096):
            T = int(rng.integers(65, 1401))
            d = int(rng.integers(40, max(41, min(5000, int(1.6e9 // (T * n))))))
            active = T if rng.integers(0, 2) else int(rng.integers(T // 2, T + 1))
            shapes.append((t, d, n, T, active, bool(rng.integers(0, 2))))
    return shapes


@pytest.mark.parametrize("t,d,n,T,active,residual", _random_prefill_shapes())
def test_prefill_on_random_shapes(ctx, t, d, n, T, active, residual):
    """Many-row projections of random shape against the oracle; rows past the active ones and
    whatever lies behind the output keep their contents."""
    from jitllm_amd import synthetic
    from jitllm_amd.projections import QuantizedBatchProjections
    say("prefill, random shape", NAMES[t], d, n, T, active, residual)
    raw = synthetic.weight(t, d, n, seed=8600 + d)
    X = synthetic.activations((T, n), seed=8700 + T)
    ref = O.matmul_batch(t, raw, X[:active], d, n)
    out = ctx.float_array(T * d + 64, fill=UNTOUCHED)
    QuantizedBatchProjections(ctx, T, n, d).projection(ctx.from_numpy(X), out, ctx.load_weight(t, raw, d, n),
                                                       n, d, residual, activeRows=active)
    ctx.sync()
    flat = out.get()
    assert np.all(flat[active * d:] == UNTOUCHED)
    got = flat[:active * d].reshape(active, d)
    want = ref.astype(np.float64) + (float(UNTOUCHED) if residual else 0.0)
    slack = abs(np.spacing(np.float32(UNTOUCHED))) / 2 if residual else 0.0
    excess = np.abs(got.astype(np.float64) - want) - slack
    assert np.all(excess <= F16_BOUND * magnitude(t, raw, X[:active], d, n)), float(excess.max())


def test_two_pass_prefill_qkv_and_gate_up(ctx):
    """The decode-once path with several weights in one call: q|k|v of unequal widths side by side,
    and gate/up interleaved by half tiles with a last tile of 8 outputs."""
    from jitllm_amd import synthetic
    from jitllm_amd.projections import QuantizedBatchProjections
    say("two-pass prefill qkv / gate_up")
    t, n, T = O.Q8_0, 256, 1024
    dims = (4096, 1024, 1000)
    raws = [synthetic.weight(t, d, n, seed=281 + i) for i, d in enumerate(dims)]
    X = synthetic.activations((T, n), seed=285)
    ws = [ctx.load_weight(t, r, d, n) for r, d in zip(raws, dims)]
    ld = sum(dims)
    out = ctx.float_array(T * ld, fill=UNTOUCHED)
    QuantizedBatchProjections(ctx, T, n, ld).fusedQKV(ctx.from_numpy(X), out, *ws)
    ctx.sync()
    got = out.get().reshape(T, ld)
    col = 0
    for raw, d in zip(raws, dims):
        ref = O.matmul_batch(t, raw, X, d, n)
        assert rel_err(got[:, col:col + d], ref, magnitude(t, raw, X, d, n)) < 2e-4
        col += d
    t, d, n, T = O.Q4_0, 7944, 256, 1024   # 256 x 256 tiles, 4 x 63 of them, the last with 8 outputs
    r1 = synthetic.weight(t, d, n, seed=291)
    r3 = synthetic.weight(t, d, n, seed=292)
    X = synthetic.activations((T, n), seed=293)
    g = O.matmul_batch(t, r1, X, d, n)
    u = O.matmul_batch(t, r3, X, d, n)
    ref = O.swiglu(g.reshape(-1), u.reshape(-1)).reshape(T, d)
    hb = ctx.float_array(T * d, fill=UNTOUCHED)
    QuantizedBatchProjections(ctx, T, n, 2 * d).gateUp(ctx.from_numpy(X), hb, ctx.load_weight(t, r1, d, n),
                                                ctx.load_weight(t, r3, d, n), n, d)
    ctx.sync()
    got = hb.get().reshape(T, d)
    mg, mu = magnitude(t, r1, X, d, n), magnitude(t, r3, X, d, n)
    bound = 2e-4 * (mg * np.abs(u) + 1.2 * mu * np.abs(g)) + 1e-6
    assert np.all(np.abs(got.astype(np.float64) - ref) <= bound)
    # gate/up on 128 x 128 tiles (9 x 20 of them: too few rows for the larger tiles), ragged rows,
    # a last tile of 54 outputs
    t, d, n, T = O.Q8_0, 1270, 512, 1100
    r1 = synthetic.weight(t, d, n, seed=295)
    r3 = synthetic.weight(t, d, n, seed=296)
    X = synthetic.activations((T, n), seed=297)
    g = O.matmul_batch(t, r1, X, d, n)
    u = O.matmul_batch(t, r3, X, d, n)
    ref = O.swiglu(g.reshape(-1), u.reshape(-1)).reshape(T, d)
    hb = ctx.float_array(T * d + 64, fill=UNTOUCHED)
    QuantizedBatchProjections(ctx, T, n, 2 * d).gateUp(ctx.from_numpy(X), hb, ctx.load_weight(t, r1, d, n),
                                                ctx.load_weight(t, r3, d, n), n, d)
    ctx.sync()
    flat = hb.get()
    assert np.all(flat[T * d:] == UNTOUCHED)
    got = flat[:T * d].reshape(T, d)
    mg, mu = magnitude(t, r1, X, d, n), magnitude(t, r3, X, d, n)
    bound = 2e-4 * (mg * np.abs(u) + 1.2 * mu * np.abs(g)) + 1e-6
    assert np.all(np.abs(got.astype(np.float64) - ref) <= bound)


@pytest.mark.parametrize("t,d,n,rows", [(O.Q4_K, 1024, 12288, 32), (O.Q8_0, 520, 4096, 64), (O.Q4_0, 4096, 6144, 9)])
def test_rows_cut_across_workgroups_are_folded_afresh_on_every_call(ctx, t, d, n, rows):
    """Rows longer than one workgroup's span are cut across workgroups; the one that finishes last
    adds the others' partial sums, which travel through the workspace.  Calls that follow one
    another without a pause, with two different inputs in turn and the same workspace, must each
    see their own partial sums -- never what an earlier call left in a cache -- and must give the
    same bits every time (the order of addition does not depend on who is last)."""
    from jitllm_amd import synthetic
    from jitllm_amd.projections import QuantizedBatchProjections
    say("folded afresh", NAMES[t], d, n, rows)
    raw = synthetic.weight(t, d, n, seed=9900 + d)
    w = ctx.load_weight(t, raw, d, n)
    Xs = [synthetic.activations((rows, n), seed=9901), synthetic.activations((rows, n), seed=9902) * np.float32(3.0)]
    xd = [ctx.from_numpy(X) for X in Xs]
    proj = QuantizedBatchProjections(ctx, rows, n, d)
    rounds = 12
    outs = [[ctx.float_array(rows * d, fill=UNTOUCHED) for _ in range(rounds)] for _ in Xs]
    for r in range(rounds):
        for i in range(2):
            proj.projection(xd[i], outs[i][r], w, n, d, False)
    ctx.sync()
    dot = O.DOT_SCALAR if t == O.Q4_K else O.DOT_VEC256
    for i, X in enumerate(Xs):
        first = outs[i][0].get().reshape(rows, d)
        err = rel_err(first, O.matmul_batch(t, raw, X, d, n, dot), magnitude(t, raw, X, d, n))
        assert err < 2e-4, err
        for r in range(1, rounds):
            assert np.array_equal(outs[i][r].get().reshape(rows, d).view(np.uint32), first.view(np.uint32)), (i, r)
    w.free()


# (type, weight rows, row length, batch, active rows, residual): 65 .. 511 rows on the
# weight-streaming kernel as 3 .. 16 row blocks -- a last block of one row, partial batches, rows cut
# across workgroups (more than 2048 columns) with up to eight blocks' partial sums in the workspace,
# the types whose other way decodes the whole weight first
MID_ROWS = [
    (O.Q8_0, 520, 2048, 65, 65, False),
    (O.Q8_0, 520, 2048, 160, 131, True),
    (O.Q4_K, 1000, 4096, 96, 96, True),
    (O.Q4_K, 264, 8192, 250, 250, False),
    (O.Q4_0, 300, 6144, 129, 100, False),
    (O.Q4_0, 2048, 256, 511, 511, True),
    (O.Q6_K, 300, 2048, 200, 170, False),
    (O.Q5_K, 520, 4096, 384, 384, True),
    (O.IQ4_XS, 264, 1024, 97, 97, False),
]


@pytest.mark.parametrize("t,d,n,batch,rows,residual", MID_ROWS)
def test_mid_row_counts_stream_their_weights(ctx, t, d, n, batch, rows, residual):
    """Calls between batched decode and prefill against the oracle; rows past the active ones and
    whatever lies behind the output keep their contents, and a second call gives the same bits."""
    from jitllm_amd import synthetic
    from jitllm_amd.projections import QuantizedBatchProjections
    say("mid row counts", t, d, n, batch, rows, residual)
    raw = synthetic.weight(t, d, n, seed=9950 + d)
    X = synthetic.activations((batch, n), seed=9951 + rows)
    ref = O.matmul_batch(t, raw, X[:rows], d, n)
    w = ctx.load_weight(t, raw, d, n)
    proj = QuantizedBatchProjections(ctx, batch, n, d)
    outs = [ctx.float_array(batch * d + 64, fill=UNTOUCHED) for _ in range(2)]
    for out in outs:
        proj.projection(ctx.from_numpy(X), out, w, n, d, residual, activeRows=rows)
    ctx.sync()
    flat = outs[0].get()
    assert np.all(flat[rows * d:] == UNTOUCHED)
    assert np.array_equal(flat.view(np.uint32), outs[1].get().view(np.uint32))
    got = flat[:rows * d].reshape(rows, d)
    want = ref.astype(np.float64) + (float(UNTOUCHED) if residual else 0.0)
    slack = abs(np.spacing(np.float32(UNTOUCHED))) / 2 if residual else 0.0
    excess = np.abs(got.astype(np.float64) - want) - slack
    assert np.all(excess <= F16_BOUND * magnitude(t, raw, X[:rows], d, n)), float(excess.max())
    w.free()


def test_mid_row_counts_gate_up_and_side_by_side_weights(ctx):
    """The other two call forms at 65 .. 511 rows: q|k|v of unequal widths side by side (five row
    blocks) and gate/up + SwiGLU (four row blocks, the last one partial), fp32 and binary16
    activations giving the same bits."""
    from jitllm_amd import synthetic
    from jitllm_amd.projections import QuantizedBatchProjections
    say("mid row counts, qkv / gate_up")
    t, n, T = O.Q8_0, 2048, 150
    dims = (1024, 256, 264)
    raws = [synthetic.weight(t, d, n, seed=9960 + i) for i, d in enumerate(dims)]
    X16 = synthetic.activations((T, n), seed=9963).astype(np.float16)
    X = X16.astype(np.float32)
    ws = [ctx.load_weight(t, r, d, n) for r, d in zip(raws, dims)]
    ld = sum(dims)
    a, b = ctx.float_array(T * ld, fill=UNTOUCHED), ctx.float_array(T * ld, fill=UNTOUCHED)
    p = QuantizedBatchProjections(ctx, T, n, ld)
    p.fusedQKV(ctx.from_numpy(X), a, *ws)
    p.fusedQKV(ctx.half_from_numpy(X16), b, *ws)
    ctx.sync()
    got = a.get().reshape(T, ld)
    assert np.array_equal(got.view(np.uint32), b.get().reshape(T, ld).view(np.uint32))
    col = 0
    for raw, d in zip(raws, dims):
        assert rel_err(got[:, col:col + d], O.matmul_batch(t, raw, X, d, n), magnitude(t, raw, X, d, n)) < F16_BOUND
        col += d
    t, d, n, T = O.Q4_K, 1000, 2048, 100
    r1, r3 = synthetic.weight(t, d, n, seed=9970), synthetic.weight(t, d, n, seed=9971)
    X = synthetic.activations((T, n), seed=9972)
    g, u = O.matmul_batch(t, r1, X, d, n), O.matmul_batch(t, r3, X, d, n)
    ref = O.swiglu(g.reshape(-1), u.reshape(-1)).reshape(T, d)
    hb = ctx.float_array(T * d + 64, fill=UNTOUCHED)
    QuantizedBatchProjections(ctx, T, n, 2 * d).gateUp(ctx.from_numpy(X), hb, ctx.load_weight(t, r1, d, n),
                                                ctx.load_weight(t, r3, d, n), n, d)
    ctx.sync()
    flat = hb.get()
    assert np.all(flat[T * d:] == UNTOUCHED)
    mg, mu = magnitude(t, r1, X, d, n), magnitude(t, r3, X, d, n)
    bound = F16_BOUND * (mg * np.abs(u) + 1.2 * mu * np.abs(g)) + 1e-6
    assert np.all(np.abs(flat[:T * d].reshape(T, d).astype(np.float64) - ref) <= bound)


MINOR = [O.Q5_K, O.Q6_K, O.Q4_1, O.Q5_0, O.IQ4_XS]


@pytest.mark.parametrize("t", MINOR)
@pytest.mark.parametrize("d,n,rows,active", [(1000, 2048, 8, 8), (1100, 4096, 32, 29), (1030, 6144, 64, 64),
                                             (1000, 14336, 17, 17), (1500, 2048, 1, 1)])
def test_minor_types_stream_their_weights_at_up_to_64_rows(ctx, t, d, n, rows, active):
    """Q6_K / Q5_K / Q4_1 / Q5_0 / IQ4_XS at up to 64 rows run the weight-streaming kernel like the
    three main types (the reference has tiled batch kernels for each: QuantizedBatchProjections.java:
    168-281): plain, residual and gate/up against the oracle, rows past the active ones untouched.
    The workspace is sized for 16 output columns -- room for partial sums, far too small for an fp16
    copy of these weights -- so a call that fell back to decoding the weights would be refused."""
    from jitllm_amd import _lib as L, synthetic
    from jitllm_amd.projections import QuantizedBatchProjections
    say("minor type, streaming", t, d, n, rows, active)
    raw = synthetic.weight(t, d, n, seed=9700 + d)
    raw_up = synthetic.weight(t, d, n, seed=9701 + d)
    X = synthetic.activations((rows, n), seed=9702 + rows)
    g = O.matmul_batch(t, raw, X[:active], d, n)
    u = O.matmul_batch(t, raw_up, X[:active], d, n)
    mg, mu = magnitude(t, raw, X[:active], d, n), magnitude(t, raw_up, X[:active], d, n)
    w, w_up = ctx.load_weight(t, raw, d, n), ctx.load_weight(t, raw_up, d, n)
    proj = QuantizedBatchProjections(ctx, rows, n, 16)
    assert proj.workspace_bytes() < 2 * d * n      # no room for 2 bytes per weight
    xd = ctx.from_numpy(X)
    start = synthetic.activations((rows, d), seed=9703)
    plain = ctx.float_array(rows * d, fill=UNTOUCHED)
    res = ctx.from_numpy(start)
    hb = ctx.float_array(rows * d, fill=UNTOUCHED)
    proj.projection(xd, plain, w, n, d, False, activeRows=active)
    proj.projection(xd, res, w, n, d, True, activeRows=active)
    proj._gemm([w, w_up], xd, hb, active, d, 0, L.JL_SWIGLU)
    ctx.sync()
    got, got_res, got_hb = (a.get().reshape(rows, d) for a in (plain, res, hb))
    assert np.all(got[active:] == UNTOUCHED) and np.all(got_hb[active:] == UNTOUCHED)
    assert np.array_equal(got_res[active:], start[active:])
    err = rel_err(got[:active], g, mg)
    assert err < F16_BOUND, err
    assert err < 3e-4, err
    assert rel_err(got_res[:active], g.astype(np.float64) + start[:active], mg + np.abs(start[:active]) * 1e-6) < 3e-4
    ref = O.swiglu(g.reshape(-1), u.reshape(-1)).reshape(active, d)
    bound = 3e-4 * (mg * np.abs(u) + 1.2 * mu * np.abs(g)) + 1e-6
    assert np.all(np.abs(got_hb[:active].astype(np.float64) - ref) <= bound)
    w.free()
    w_up.free()


def _random_minor_shapes():
    """Seeded shapes for the five minor types across the streaming kernel's geometries: row lengths
    it takes for each type (a span must be a whole number of 16-byte pieces: Q6_K rows of a multiple
    of 2048 columns, IQ4_XS of 512, the others of 256) and some it does not (those fall back to the
    decode-once path, which the ordinary workspace holds), 1 .. 64 rows, partial batches."""
    rng = np.random.default_rng(20261127)
    shapes = []
    for t in MINOR:
        for n in (256, 512, 1280, 2048, 2304, 4096, 6144, 8192):
            rows = int(rng.choice([1, 2, 7, 8, 9, 16, 17, 31, 32, 33, 48, 64]))
            d = int(rng.integers(1, 260))
            active = rows if rng.integers(0, 2) else int(rng.integers(1, rows + 1))
            shapes.append((t, d, n, rows, active))
    return shapes


@pytest.mark.parametrize("t,d,n,rows,active", _random_minor_shapes())
def test_minor_types_on_random_shapes(ctx, t, d, n, rows, active):
    from jitllm_amd import _lib as L, synthetic
    from jitllm_amd.projections import QuantizedBatchProjections
    say("minor type, random shape", t, d, n, rows, active)
    raw = synthetic.weight(t, d, n, seed=9850 + d)
    raw_up = synthetic.weight(t, d, n, seed=9851 + d)
    X = synthetic.activations((rows, n), seed=9852 + n)
    g = O.matmul_batch(t, raw, X[:active], d, n)
    u = O.matmul_batch(t, raw_up, X[:active], d, n)
    mg, mu = magnitude(t, raw, X[:active], d, n), magnitude(t, raw_up, X[:active], d, n)
    w, w_up = ctx.load_weight(t, raw, d, n), ctx.load_weight(t, raw_up, d, n)
    proj = QuantizedBatchProjections(ctx, rows, n, 2 * d)
    xd = ctx.from_numpy(X)
    plain = ctx.float_array(rows * d, fill=UNTOUCHED)
    res = ctx.float_array(rows * d, fill=UNTOUCHED)
    hb = ctx.float_array(rows * d, fill=UNTOUCHED)
    proj.projection(xd, plain, w, n, d, False, activeRows=active)
    proj.projection(xd, res, w, n, d, True, activeRows=active)
    proj._gemm([w, w_up], xd, hb, active, d, 0, L.JL_SWIGLU)
    ctx.sync()
    got, got_res, got_hb = (a.get().reshape(rows, d) for a in (plain, res, hb))
    for a in (got, got_res, got_hb):
        assert np.all(a[active:] == UNTOUCHED)
    assert rel_err(got[:active], g, mg) < 5e-4
    assert rel_err(got_res[:active], g.astype(np.float64) + float(UNTOUCHED), mg + 12345.5 * 6e-8) < 5e-4
    ref = O.swiglu(g.reshape(-1), u.reshape(-1)).reshape(active, d)
    bound = 5e-4 * (mg * np.abs(u) + 1.2 * mu * np.abs(g)) + 1e-6
    assert np.all(np.abs(got_hb[:active].astype(np.float64) - ref) <= bound)
    w.free()
    w_up.free()


@pytest.mark.parametrize("t", MINOR)
def test_minor_type_super_blocks_with_extreme_scales(ctx, t):
    """Scales at their extremes: every sub-block scale / minimum field at its largest, the signed
    Q6_K scales at -128 (where scale x quant passes 2048 and a fragment is rounded), quants at both
    ends -- against the oracle at 9 rows."""
    from jitllm_amd import synthetic
    from jitllm_amd.projections import QuantizedBatchProjections
    say("minor type, extreme scales", t)
    d, n, rows = 48, 2048, 9
    raw = synthetic.weight(t, d, n, seed=9800).copy()
    bb, be = O.block_bytes(t), O.block_elems(t)
    blocks = raw.reshape(-1, bb)
    rng = np.random.default_rng(9801)
    pick = rng.random(blocks.shape[0]) < 0.5
    if t == O.Q6_K:
        blocks[pick, 192:208] = np.where(rng.random((int(pick.sum()), 16)) < 0.5, 0x80, 0x7F).astype(np.uint8)
        blocks[pick, :192] = np.where(rng.random((int(pick.sum()), 192)) < 0.5, 0x00, 0xFF).astype(np.uint8)
    elif t == O.Q5_K:
        blocks[pick, 4:16] = 0xFF
        blocks[pick, 16:] = np.where(rng.random((int(pick.sum()), bb - 16)) < 0.5, 0x00, 0xFF).astype(np.uint8)
    elif t == O.IQ4_XS:
        blocks[pick, 2:8] = np.where(rng.random((int(pick.sum()), 6)) < 0.5, 0x00, 0xFF).astype(np.uint8)
        blocks[pick, 8:] = np.where(rng.random((int(pick.sum()), bb - 8)) < 0.5, 0x00, 0x77).astype(np.uint8)
    else:   # Q4_1 (d, m | 16 B), Q5_0 (d | 4 B | 16 B): quants and fifth bits at both ends
        head = 4 if t == O.Q4_1 else 2
        blocks[pick, head:] = np.where(rng.random((int(pick.sum()), bb - head)) < 0.5, 0x00, 0xFF).astype(np.uint8)
    raw = blocks.reshape(-1)
    X = synthetic.activations((rows, n), seed=9802)
    ref = O.matmul_batch(t, raw, X, d, n)
    out = ctx.float_array(rows * d, fill=UNTOUCHED)
    QuantizedBatchProjections(ctx, rows, n, 16).projection(ctx.from_numpy(X), out, ctx.load_weight(t, raw, d, n), n, d, False)
    ctx.sync()
    err = rel_err(out.get().reshape(rows, d), ref, magnitude(t, raw, X, d, n))
    assert err < 5e-4, err


@pytest.mark.parametrize("t", MINOR)
@pytest.mark.parametrize("d,n,T,residual", [(300, 512, 8, False), (1000, 2048, 100, True), (4096, 256, 600, False)])
def test_k_quant_batched_rows_take_the_decode_once_path(ctx, t, d, n, T, residual):
    """A Q6_K / Q5_K / Q4_1 / Q5_0 / IQ4_XS weight has no decode-in-the-loop GEMM: batched calls of
    more than 64 rows (and shapes the weight-streaming kernel does not take) decode it to fp16 into
    the workspace and run the fp16 GEMM; partial batches leave the rest alone."""
    from jitllm_amd import synthetic
    from jitllm_amd.projections import QuantizedBatchProjections
    say("k-quant batched", t, d, n, T, residual)
    raw = synthetic.weight(t, d, n, seed=9300 + d)
    X = synthetic.activations((T, n), seed=9400 + T)
    active = T - 3
    ref = O.matmul_batch(t, raw, X, d, n)
    out = ctx.float_array(T * d, fill=UNTOUCHED)
    proj = QuantizedBatchProjections(ctx, T, n, d)
    proj.projection(ctx.from_numpy(X), out, ctx.load_weight(t, raw, d, n), n, d, residual, activeRows=active)
    ctx.sync()
    got = out.get().reshape(T, d)
    assert np.all(got[active:] == UNTOUCHED)
    want = ref.astype(np.float64) + (float(UNTOUCHED) if residual else 0.0)
    slack = abs(np.spacing(np.float32(UNTOUCHED))) / 2 if residual else 0.0
    excess = np.abs(got[:active].astype(np.float64) - want[:active]) - slack
    assert np.all(excess <= 5e-4 * magnitude(t, raw, X, d, n)[:active]), float(excess.max())


def test_q6_k_batched_gate_up(ctx):
    from jitllm_amd import synthetic
    from jitllm_amd.projections import QuantizedBatchProjections
    say("q6_K batched gate_up")
    t, d, n, T = O.Q6_K, 200, 512, 40
    r1 = synthetic.weight(t, d, n, seed=9501)
    r3 = synthetic.weight(t, d, n, seed=9502)
    X = synthetic.activations((T, n), seed=9503)
    g = O.matmul_batch(t, r1, X, d, n)
    u = O.matmul_batch(t, r3, X, d, n)
    ref = O.swiglu(g.reshape(-1), u.reshape(-1)).reshape(T, d)
    hb = ctx.float_array(T * d, fill=UNTOUCHED)
    # (the host mirror keeps the reference's rule that gate/up is fused for Q8_0 / Q4_0 / Q4_K
    # pairs only; the library's jl_gemm takes the Q6_K pair, so it is called directly)
    from jitllm_amd import _lib as L
    proj = QuantizedBatchProjections(ctx, T, n, 2 * d)
    assert not proj.fusedGateUp(ctx.load_weight(t, r1, d, n), ctx.load_weight(t, r3, d, n))
    proj._gemm([ctx.load_weight(t, r1, d, n), ctx.load_weight(t, r3, d, n)], ctx.from_numpy(X), hb, T, d, 0,
               L.JL_SWIGLU)
    ctx.sync()
    got = hb.get().reshape(T, d)
    mg, mu = magnitude(t, r1, X, d, n), magnitude(t, r3, X, d, n)
    bound = 5e-4 * (mg * np.abs(u) + 1.2 * mu * np.abs(g)) + 1e-6
    assert np.all(np.abs(got.astype(np.float64) - ref) <= bound)


def test_resident_fp16_copy_gives_the_same_bits(ctx):
    """The reference's residency choice: the decoded copy is kept in a caller-owned buffer and
    decoded on the first call only.  Same results as without, on the first call, on the second
    (no decode), and after the row count -- hence the gate/up layout -- changes."""
    from jitllm_amd import synthetic
    from jitllm_amd.projections import QuantizedBatchProjections
    say("resident copy")
    t, d, n = O.Q8_0, 5800, 256
    raw = synthetic.weight(t, d, n, seed=9601)
    w = ctx.load_weight(t, raw, d, n)
    r1, r3 = synthetic.weight(t, 8200, n, seed=9602), synthetic.weight(t, 8200, n, seed=9603)
    w1, w3 = ctx.load_weight(t, r1, 8200, n), ctx.load_weight(t, r3, 8200, n)
    T = 2048
    X = ctx.from_numpy(synthetic.activations((T, n), seed=9604))
    plain = QuantizedBatchProjections(ctx, T, n, 2 * 8200)
    kept = QuantizedBatchProjections(ctx, T, n, 2 * 8200, resident=True)
    def run(p, rows):
        out = ctx.float_array(T * d, fill=UNTOUCHED)
        hb = ctx.float_array(T * 8200, fill=UNTOUCHED)
        p.projection(X, out, w, n, d, False, activeRows=rows)
        p.gateUp(X, hb, w1, w3, n, 8200, activeRows=rows)
        ctx.sync()
        return out.get(), hb.get()
    for rows in (2048, 2048, 1024, 2048, 700):      # 1024 rows pick another column tile for gate/up
        a, b = run(plain, rows), run(kept, rows)
        assert np.array_equal(a[0].view(np.uint32), b[0].view(np.uint32)), rows
        assert np.array_equal(a[1].view(np.uint32), b[1].view(np.uint32)), rows
    assert len(kept._copies) == 2


@pytest.mark.parametrize("t,d,n,rows,residual", [(O.Q8_0, 16384, 2048, 300, False), (O.Q4_K, 12288, 4096, 200, True)])
def test_kept_copy_at_mid_row_counts(ctx, t, d, n, rows, residual):
    """128 .. 511 rows over a kept fp16 copy run the plain fp16 GEMM where the call without one
    decodes in its loop: the same fp16 products in another order of addition.  Both against the
    oracle on the weight's first and last rows, and against each other; the second call (no decode)
    gives the first one's bits."""
    from jitllm_amd import synthetic
    from jitllm_amd.projections import QuantizedBatchProjections
    say("kept copy, mid rows", t, d, n, rows, residual)
    raw = synthetic.weight(t, d, n, seed=9650)
    w = ctx.load_weight(t, raw, d, n)
    X = synthetic.activations((rows, n), seed=9651)
    start = synthetic.activations((rows, d), seed=9652) if residual else np.full((rows, d), UNTOUCHED, np.float32)
    plain = QuantizedBatchProjections(ctx, rows, n, d)
    kept = QuantizedBatchProjections(ctx, rows, n, d, resident=True)
    outs = [ctx.from_numpy(start) for _ in range(3)]
    plain.projection(ctx.from_numpy(X), outs[0], w, n, d, residual)
    kept.projection(ctx.from_numpy(X), outs[1], w, n, d, residual)
    kept.projection(ctx.from_numpy(X), outs[2], w, n, d, residual)
    ctx.sync()
    a, b, c = (o.get().reshape(rows, d) for o in outs)
    assert np.array_equal(b.view(np.uint32), c.view(np.uint32))
    row_bytes = raw.size // d
    edge = 96
    for cols, part in ((slice(0, edge), raw[:edge * row_bytes]), (slice(d - edge, d), raw[(d - edge) * row_bytes:])):
        ref = O.matmul_batch(t, part, X, edge, n).astype(np.float64) + (start[:, cols] if residual else 0.0)
        mag = magnitude(t, part, X, edge, n) + (np.abs(start[:, cols]) * 1e-6 if residual else 0.0)
        assert rel_err(a[:, cols], ref, mag) < F16_BOUND
        assert rel_err(b[:, cols], ref, mag) < F16_BOUND
        assert rel_err(b[:, cols], a[:, cols].astype(np.float64), mag) < 1e-5
    w.free()


@pytest.mark.parametrize("t,d,n,batch,rows,tight", [(O.Q6_K, 5870, 768, 243, 243, False), (O.Q6_K, 3554, 1024, 345, 155, False),
                                                    (O.Q6_K, 5870, 768, 243, 243, True), (O.Q8_0, 4000, 1024, 130, 130, True),
                                                    (O.Q4_K, 1500, 2048, 600, 600, True)])
def test_kept_copy_of_a_narrow_projection_cuts_k_only_where_the_workspace_has_room(ctx, t, d, n, batch, rows, tight):
    """A narrow projection over a kept copy would cut K and fold partial sums from the workspace:
    with the workspace the size query gives it does, with the least workspace a call may bring
    (``tight``: the activations' region only) it keeps K whole -- and a type that has no kernel but
    the decode-once one is served either way instead of refused."""
    from jitllm_amd import synthetic
    from jitllm_amd.projections import QuantizedBatchProjections
    say("kept copy, narrow projection", t, d, n, batch, rows, tight)
    raw = synthetic.weight(t, d, n, seed=9670 + d)
    w = ctx.load_weight(t, raw, d, n)
    X = synthetic.activations((batch, n), seed=9671)
    kept = QuantizedBatchProjections(ctx, batch, n, 0 if tight else d, resident=True)
    outs = [ctx.float_array(batch * d, fill=UNTOUCHED) for _ in range(2)]
    for out in outs:
        kept.projection(ctx.from_numpy(X), out, w, n, d, False, activeRows=rows)
    ctx.sync()
    a, b = (o.get().reshape(batch, d) for o in outs)
    assert np.array_equal(a.view(np.uint32), b.view(np.uint32))
    assert np.all(a[rows:] == UNTOUCHED)
    row_bytes = raw.size // d
    edge = 96
    for cols, part in ((slice(0, edge), raw[:edge * row_bytes]), (slice(d - edge, d), raw[(d - edge) * row_bytes:])):
        ref = O.matmul_batch(t, part, X[:rows], edge, n)
        assert rel_err(a[:rows, cols], ref, magnitude(t, part, X[:rows], edge, n)) < F16_BOUND
    w.free()


def test_kept_copy_gate_up_at_mid_row_counts(ctx):
    """gate/up + SwiGLU at 300 rows over a kept copy (the plain fp16 GEMM on interleaved half tiles),
    fp32 result and binary16 result, against the oracle on the first and last outputs; then 40 rows
    with the same projections, which stream the weights and leave the kept copy alone."""
    from jitllm_amd import _lib as L, synthetic
    from jitllm_amd.projections import QuantizedBatchProjections
    say("kept copy, mid rows, gate/up")
    t, d, n, rows = O.Q8_0, 8192, 2048, 300
    r1, r3 = synthetic.weight(t, d, n, seed=9660), synthetic.weight(t, d, n, seed=9661)
    w1, w3 = ctx.load_weight(t, r1, d, n), ctx.load_weight(t, r3, d, n)
    X16 = synthetic.activations((rows, n), seed=9662).astype(np.float16)
    X = X16.astype(np.float32)
    kept = QuantizedBatchProjections(ctx, rows, n, 2 * d, resident=True)
    edge, row_bytes = 64, r1.size // d

    def check(got, active):
        for cols in (slice(0, edge), slice(d - edge, d)):
            lo = cols.start * row_bytes
            g = O.matmul_batch(t, r1[lo:lo + edge * row_bytes], X[:active], edge, n)
            u = O.matmul_batch(t, r3[lo:lo + edge * row_bytes], X[:active], edge, n)
            want = O.swiglu(g.reshape(-1), u.reshape(-1)).reshape(active, edge)
            mg = magnitude(t, r1[lo:lo + edge * row_bytes], X[:active], edge, n)
            mu = magnitude(t, r3[lo:lo + edge * row_bytes], X[:active], edge, n)
            bound = F16_BOUND * (mg * np.abs(u) + 1.2 * mu * np.abs(g)) + 1e-6
            assert np.all(np.abs(got[:active, cols].astype(np.float64) - want) <= bound)

    for active in (rows, 40):
        h32 = ctx.float_array(rows * d, fill=UNTOUCHED)
        h16 = ctx.half_from_numpy(np.full(rows * d, 7.5, dtype=np.float16))
        kept._gemm([w1, w3], ctx.half_from_numpy(X16), h32, active, d, 0, L.JL_SWIGLU)
        kept._gemm([w1, w3], ctx.half_from_numpy(X16), h16, active, d, 0, L.JL_SWIGLU)
        ctx.sync()
        a, b = h32.get().reshape(rows, d), h16.get().reshape(rows, d)
        check(a, active)
        assert np.array_equal(b[:active].view(np.uint16), a[:active].astype(np.float16).view(np.uint16))
        assert np.all(a[active:] == UNTOUCHED) and np.all(b[active:] == np.float16(7.5))


@pytest.mark.parametrize("rows", [7, 40, 200, 700])
@pytest.mark.parametrize("resident", [False, True])
def test_weights_of_different_types_side_by_side(ctx, rows, resident):
    """q | k | v as a "Q4_K_M" file holds them -- q and k in Q4_K, v in Q6_K -- in one call, and a
    Q5_0 gate with an IQ4_XS up weight: each weight is decoded by its own type (the reference's
    prefill projections pick the decode task per weight, FP16Projections.java:250-330), at every
    row count, with and without a kept copy, fp32 and binary16 activations giving the same bits."""
    from jitllm_amd import _lib as L, synthetic
    from jitllm_amd.projections import QuantizedBatchProjections
    say("mixed types side by side", rows, resident)
    n = 2048
    types, dims = (O.Q4_K, O.Q4_K, O.Q6_K), (1000, 264, 250)
    raws = [synthetic.weight(t, d, n, seed=9700 + i) for i, (t, d) in enumerate(zip(types, dims))]
    ws = [ctx.load_weight(t, r, d, n) for t, r, d in zip(types, raws, dims)]
    X16 = synthetic.activations((rows, n), seed=9703).astype(np.float16)
    X = X16.astype(np.float32)
    ld = sum(dims) + 9
    proj = QuantizedBatchProjections(ctx, rows, n, sum(dims), resident=resident)
    outs = [ctx.float_array(rows * ld, fill=UNTOUCHED) for _ in range(3)]
    proj._gemm(ws, ctx.from_numpy(X), outs[0], rows, ld, 5, L.JL_STORE)
    proj._gemm(ws, ctx.half_from_numpy(X16), outs[1], rows, ld, 5, L.JL_STORE)
    proj._gemm(ws, ctx.from_numpy(X), outs[2], rows, ld, 5, L.JL_STORE)     # (a kept copy: no decode this time)
    ctx.sync()
    got = outs[0].get().reshape(rows, ld)
    for other in outs[1:]:
        assert np.array_equal(got.view(np.uint32), other.get().reshape(rows, ld).view(np.uint32))
    assert np.all(got[:, :5] == UNTOUCHED) and np.all(got[:, 5 + sum(dims):] == UNTOUCHED)
    col = 5
    for t, raw, d in zip(types, raws, dims):
        assert rel_err(got[:, col:col + d], O.matmul_batch(t, raw, X, d, n), magnitude(t, raw, X, d, n)) < F16_BOUND
        col += d
    # gate / up of different types: not a pair the reference fuses, one call here all the same
    d = 520
    r1, r3 = synthetic.weight(O.Q5_0, d, n, seed=9710), synthetic.weight(O.IQ4_XS, d, n, seed=9711)
    g, u = O.matmul_batch(O.Q5_0, r1, X, d, n), O.matmul_batch(O.IQ4_XS, r3, X, d, n)
    ref = O.swiglu(g.reshape(-1), u.reshape(-1)).reshape(rows, d)
    hb = ctx.float_array(rows * d + 64, fill=UNTOUCHED)
    pair = QuantizedBatchProjections(ctx, rows, n, 2 * d, resident=resident)
    w1, w3 = ctx.load_weight(O.Q5_0, r1, d, n), ctx.load_weight(O.IQ4_XS, r3, d, n)
    assert not pair.fusedGateUp(w1, w3)
    pair.gateUp(ctx.from_numpy(X), hb, w1, w3, n, d)
    ctx.sync()
    flat = hb.get()
    assert np.all(flat[rows * d:] == UNTOUCHED)
    mg, mu = magnitude(O.Q5_0, r1, X, d, n), magnitude(O.IQ4_XS, r3, X, d, n)
    bound = F16_BOUND * (mg * np.abs(u) + 1.2 * mu * np.abs(g)) + 1e-6
    assert np.all(np.abs(flat[:rows * d].reshape(rows, d).astype(np.float64) - ref) <= bound)


@pytest.mark.parametrize("rows,n,stride", [(1, 1000, 1000), (8, 128256, 128256), (64, 32000, 32003), (40, 5, 9),
                                           (300, 4097, 4100)])
def test_argmax_of_every_row_of_batched_logits(ctx, rows, n, stride):
    """batchedArgmaxLogits: one token per row in one launch, the host scan's rule on ties and NaN
    (first maximum; a NaN at element 0 wins, elsewhere never; all -inf gives 0); row strides that
    leave the rows off a 16-byte boundary; rows past the active ones keep their token."""
    from jitllm_amd.projections import QuantizedBatchProjections
    say("argmax rows", rows, n, stride)
    rng = np.random.default_rng(9800 + rows)
    v = rng.standard_normal((rows + 2, stride)).astype(np.float32)
    v[:, n:] = 1e30                                        # what lies between the rows is not looked at
    for b in range(rows):
        v[b, rng.integers(0, n, size=3)] = 7.0             # the maximum three times: the first one counts
    if rows > 3 and n > 4:
        v[1, :n] = -np.inf
        v[2, 0] = np.nan
        v[3, n // 2] = np.nan
    logits = ctx.from_numpy(v.reshape(-1))
    tokens = ctx.raw_buffer(4 * (rows + 2))
    tokens.upload(np.full(rows + 2, -5, dtype=np.int32))
    QuantizedBatchProjections(ctx, rows + 2, 256, 256).argmaxLogits(logits, n, tokens, activeRows=rows, rowStride=stride)
    ctx.sync()
    got = tokens.download(np.int32, rows + 2)
    assert np.all(got[rows:] == -5)
    for b in range(rows):
        assert int(got[b]) == O.argmax(v[b, :n]), b


def test_huge_activation_rows_stay_finite(ctx):
    """Rows far outside fp16's range are rescaled by a power of two, not turned into infinities."""
    from jitllm_amd import synthetic
    from jitllm_amd.projections import QuantizedBatchProjections
    say("batched huge rows")
    d, n, B = 128, 1024, 4
    raw = synthetic.weight(O.Q8_0, d, n, seed=95)
    X = synthetic.activations((B, n), seed=96)
    X[1] *= 1e7
    X[2] *= 1e-6
    ref = O.matmul_batch(O.Q8_0, raw, X, d, n)
    out = ctx.float_array(B * d)
    QuantizedBatchProjections(ctx, B, n, d).projection(ctx.from_numpy(X), out,
                                                    ctx.load_weight(O.Q8_0, raw, d, n), n, d, False)
    ctx.sync()
    got = out.get().reshape(B, d)
    assert np.all(np.isfinite(got))
    err = rel_err(got, ref, magnitude(O.Q8_0, raw, X, d, n))
    assert err < 2e-4, err


def test_batched_errors(ctx):
    import ctypes as C
    from jitllm_amd import _lib as L, synthetic
    say("batched errors")
    lib = L.load()
    w = ctx.load_weight(O.Q4_K, synthetic.weight(O.Q4_K, 64, 256, 1), 64, 256)
    x, o = ctx.float_array(4 * 256, 0.0), ctx.float_array(4 * 64, 0.0)
    arr = (C.c_void_p * 1)(w.handle)
    ws = ctx.raw_buffer(1 << 20)
    st = lib.jl_gemm(ctx.handle, arr, 1, x.ptr, o.ptr, 4, 4, 64, 0, L.JL_STORE, L.JL_MATH_INT8, ws.ptr, ws.nbytes)
    assert st == L.JL_ERR_UNSUPPORTED and b"Q4_K" in lib.jl_last_error()
    st = lib.jl_gemm(ctx.handle, arr, 1, x.ptr, o.ptr, 4, 4, 64, 0, L.JL_STORE, L.JL_MATH_F16, ws.ptr, 16)
    assert st == L.JL_ERR_WORKSPACE
    st = lib.jl_gemm(ctx.handle, arr, 1, x.ptr, o.ptr, 4, 5, 64, 0, L.JL_STORE, L.JL_MATH_F16, ws.ptr, ws.nbytes)
    assert st == L.JL_ERR_INVALID
    st = lib.jl_gemm(ctx.handle, arr, 1, x.ptr, o.ptr, 4, 4, 32, 0, L.JL_STORE, L.JL_MATH_F16, ws.ptr, ws.nbytes)
    assert st == L.JL_ERR_INVALID and b"ldo" in lib.jl_last_error()
    # the int8 mode multiplies the raw blocks: no mixed types there
    w8 = ctx.load_weight(O.Q8_0, synthetic.weight(O.Q8_0, 64, 256, 2), 64, 256)
    w4 = ctx.load_weight(O.Q4_0, synthetic.weight(O.Q4_0, 64, 256, 3), 64, 256)
    two = (C.c_void_p * 2)(w8.handle, w4.handle)
    o2 = ctx.float_array(4 * 128, 0.0)
    st = lib.jl_gemm(ctx.handle, two, 2, x.ptr, o2.ptr, 4, 4, 128, 0, L.JL_STORE, L.JL_MATH_INT8, ws.ptr, ws.nbytes)
    assert st == L.JL_ERR_UNSUPPORTED and b"mixed weight types Q8_0 and Q4_0" in lib.jl_last_error()


@pytest.mark.parametrize("t,residual", [(O.Q8_0, False), (O.Q4_K, True)])
def test_with_k_kept_whole_a_row_does_not_depend_on_the_chunk(ctx, t, residual):
    """jl_context_set_split_k(0) is the reference's -Djitllm.prefill.splitK=false (SplitKGemm.java:40-42):
    a 2048-wide projection of a 512-row chunk, which otherwise cuts K into runs and adds their partial
    sums afterwards, then gives each of its rows bit for bit what the same row gets in a 2048-row
    chunk, whose K is whole anyway; with the switch on the two differ in their last bits.  The oracle
    holds either way."""
    from jitllm_amd import synthetic
    from jitllm_amd.projections import QuantizedBatchProjections
    d, n, small, large = 2048, 2048, 512, 2048
    say("K kept whole", t, residual)
    raw = synthetic.weight(t, d, n, seed=9680)
    w = ctx.load_weight(t, raw, d, n)
    X = synthetic.activations((large, n), seed=9681)
    base = synthetic.activations((large, d), seed=9682) if residual else None

    def run(rows):
        proj = QuantizedBatchProjections(ctx, rows, n, d)
        out = ctx.from_numpy(base[:rows].reshape(-1).copy()) if residual else ctx.float_array(rows * d, fill=UNTOUCHED)
        proj.projection(ctx.from_numpy(X[:rows]), out, w, n, d, residual)
        ctx.sync()
        got = out.get().reshape(rows, d)
        out.free()
        proj.workspace.free()
        return got

    try:
        ctx.set_split_k(False)
        whole_small, whole_large = run(small), run(large)
        ctx.set_split_k(True)
        cut_small = run(small)
    finally:
        ctx.set_split_k(True)
    assert np.array_equal(whole_small.view(np.uint32), whole_large[:small].view(np.uint32))
    assert not np.array_equal(cut_small.view(np.uint32), whole_small.view(np.uint32))
    edge, row_bytes = 64, raw.size // d
    for got in (whole_small, cut_small):
        ref = O.matmul_batch(t, raw[:edge * row_bytes], X[:small], edge, n)
        delta = got[:, :edge] - (base[:small, :edge] if residual else 0.0)
        assert rel_err(delta, ref, magnitude(t, raw[:edge * row_bytes], X[:small], edge, n)) < F16_BOUND
    w.free()


def test_two_contexts_on_two_host_threads():
    """Two host threads, a context (and stream) each, on the one device at the same time -- a second
    session beside the first.  Every call's result is bit for bit what the same thread got the first
    time, and the first meets the oracle: contexts share nothing that a call writes (their scratch,
    arrival counters and workspaces are their own; the once-per-kernel set-up is guarded)."""
    import threading

    from jitllm_amd import synthetic
    from jitllm_amd.projections import QuantizedBatchProjections, QuantizedProjections, TornadoWorkspace
    from jitllm_amd.runtime import Context
    say("two contexts, two threads")
    t, d, n = O.Q4_K, 1536, 2048
    raws = [synthetic.weight(t, d, n, seed=9700 + i) for i in range(2)]
    X = synthetic.activations((600, n), seed=9702)
    failures = []

    def session(index):
        try:
            with Context(0) as c:
                w = c.load_weight(t, raws[index], d, n)
                single = QuantizedProjections(c, TornadoWorkspace())
                dx = c.from_numpy(X[0])
                first = {}
                for it in range(40):
                    for rows in (1, 40, 200, 600):
                        if rows == 1:
                            out = c.float_array(d, fill=UNTOUCHED)
                            single.floatMatvec(dx, out, w, n, d)
                        else:
                            proj = QuantizedBatchProjections(c, rows, n, d)
                            out = c.float_array(rows * d, fill=UNTOUCHED)
                            proj.projection(c.from_numpy(X[:rows]), out, w, n, d, False)
                        c.sync()
                        got = out.get().reshape(rows, d)
                        out.free()
                        if rows != 1:
                            proj.workspace.free()
                        if it == 0:
                            first[rows] = got
                            ref = O.matmul_batch(t, raws[index][:64 * (raws[index].size // d)], X[:rows], 64, n)
                            mag = magnitude(t, raws[index][:64 * (raws[index].size // d)], X[:rows], 64, n)
                            assert rel_err(got[:, :64], ref, mag) < F16_BOUND, (index, rows)
                        else:
                            assert np.array_equal(got.view(np.uint32), first[rows].view(np.uint32)), (index, it, rows)
                w.free()
        except BaseException as e:   # noqa: BLE001 -- handed to the main thread
            failures.append((index, repr(e)))

    threads = [threading.Thread(target=session, args=(i,)) for i in range(2)]
    for th in threads:
        th.start()
    for th in threads:
        th.join()
    assert not failures, failures


@pytest.mark.parametrize("t,d,n,rows,active,residual,half", [
    (O.Q4_K, 520, 11008, 8, 8, False, False), (O.Q8_0, 264, 11008, 32, 29, True, False),
    (O.Q4_0, 136, 18944, 64, 64, True, False), (O.Q4_K, 100, 18944, 17, 17, False, True),
    (O.Q5_K, 72, 11008, 40, 33, True, False), (O.Q8_0, 48, 2816, 8, 5, False, False),
    (O.Q4_K, 36, 4864, 64, 64, True, True), (O.Q6_K, 24, 11008, 8, 8, True, False),
    (O.Q4_K, 520, 11008, 96, 96, True, False), (O.Q8_0, 264, 18944, 200, 150, False, False),
    (O.Q4_0, 4096, 11008, 384, 384, True, False)])
def test_row_lengths_with_no_equal_spans(ctx, t, d, n, rows, active, residual, half):
    """11 008 columns are 43 blocks of 256 and 18 944 are 74: no cut into equal spans of up to eight
    blocks but spans of one or two.  Batched decode and short prompts (up to 511 rows) take such a row as
    its whole eights of blocks and, in a second launch that adds to the first, the rest; here against the
    oracle on every output (the largest case: on the first 64), for
    fp32 and binary16 activations, partial batches, stored and accumulated results (Q6_K, whose blocks
    start on a 16-byte boundary only every eighth, keeps the path it had)."""
    from jitllm_amd import synthetic
    from jitllm_amd.projections import QuantizedBatchProjections
    say("rows without equal spans", t, d, n, rows, active, residual, half)
    raw = synthetic.weight(t, d, n, seed=9910 + d)
    w = ctx.load_weight(t, raw, d, n)
    X = synthetic.activations((rows, n), seed=9911)
    if half:
        X = X.astype(np.float16).astype(np.float32)
    base = synthetic.activations((rows, d), seed=9912) if residual else np.full((rows, d), UNTOUCHED, np.float32)
    proj = QuantizedBatchProjections(ctx, rows, n, d)
    dx = ctx.half_from_numpy(X.astype(np.float16)) if half else ctx.from_numpy(X)
    outs = []
    for _ in range(2):
        out = ctx.from_numpy(base.reshape(-1).copy())
        proj.projection(dx, out, w, n, d, residual, activeRows=active)
        ctx.sync()
        outs.append(out.get().reshape(rows, d))
        out.free()
    got = outs[0]
    assert np.array_equal(got.view(np.uint32), outs[1].view(np.uint32))
    assert np.array_equal(got[active:], base[active:])
    cols = min(d, 64) if d > 1024 else d
    part = raw[:cols * (raw.size // d)]
    ref = O.matmul_batch(t, part, X[:active], cols, n)
    delta = got[:active, :cols] - (base[:active, :cols] if residual else 0.0)
    assert rel_err(delta, ref, magnitude(t, part, X[:active], cols, n) + (np.abs(base[:active, :cols]) * 1e-6 if residual else 0.0)) < F16_BOUND
    proj.workspace.free()
    w.free()


@pytest.mark.parametrize("t,n", [(O.Q8_0, 896), (O.Q4_0, 896), (O.Q8_0, 1600), (O.Q5_0, 2112)])
@pytest.mark.parametrize("rows", [3, 64, 200, 640])
def test_row_lengths_that_are_not_whole_256_column_blocks(ctx, t, n, rows):
    """896 columns (the width of the smallest Qwen2.5) are whole 64-column steps but three and a half
    256-column blocks: such rows take the decode-once path at every row count -- a projection, q | k
    side by side and gate/up + SwiGLU against the oracle."""
    from jitllm_amd import synthetic
    from jitllm_amd.projections import QuantizedBatchProjections
    say("rows that are no whole 256-column blocks", t, n, rows)
    d, dk = 328, 136
    r1, r3 = synthetic.weight(t, d, n, seed=9920), synthetic.weight(t, d, n, seed=9921)
    rk = synthetic.weight(t, dk, n, seed=9922)
    w1, w3, wk = ctx.load_weight(t, r1, d, n), ctx.load_weight(t, r3, d, n), ctx.load_weight(t, rk, dk, n)
    X = synthetic.activations((rows, n), seed=9923)
    proj = QuantizedBatchProjections(ctx, rows, n, 2 * d)
    dx = ctx.from_numpy(X)
    out, hb = ctx.float_array(rows * d, fill=UNTOUCHED), ctx.float_array(rows * d, fill=UNTOUCHED)
    side = ctx.float_array(rows * (d + 2 * dk), fill=UNTOUCHED)
    proj.projection(dx, out, w1, n, d, False)
    proj.fusedQKV(dx, side, w1, wk, wk)
    proj.gateUp(dx, hb, w1, w3, n, d)
    ctx.sync()
    g, u = O.matmul_batch(t, r1, X, d, n), O.matmul_batch(t, r3, X, d, n)
    mg, mu = magnitude(t, r1, X, d, n), magnitude(t, r3, X, d, n)
    assert rel_err(out.get().reshape(rows, d), g, mg) < F16_BOUND
    s = side.get().reshape(rows, d + 2 * dk)
    assert rel_err(s[:, :d], g, mg) < F16_BOUND
    kref, mk = O.matmul_batch(t, rk, X, dk, n), magnitude(t, rk, X, dk, n)
    assert rel_err(s[:, d:d + dk], kref, mk) < F16_BOUND and rel_err(s[:, d + dk:], kref, mk) < F16_BOUND
    got = hb.get().reshape(rows, d).astype(np.float64)
    g64, u64 = g.astype(np.float64), u.astype(np.float64)
    want = g64 / (1.0 + np.exp(-g64)) * u64
    bound = F16_BOUND * (mg * (np.abs(u64) + mu) + mu * np.abs(g64)) + 1e-6
    assert np.all(np.abs(got - want) <= bound)
    for w in (w1, w3, wk):
        w.free()
    proj.workspace.free()


@pytest.mark.parametrize("rows", [8, 64, 200])
def test_mixed_types_side_by_side_below_512_rows_are_their_runs(ctx, rows):
    """A "Q4_K_M" q | k | v (q and k in Q4_K, v in Q6_K) at a few rows is made one run of equal types at a
    time, each through the kernels its type has: the result is bit for bit what the two calls -- q | k,
    then v beside them -- leave, and meets the oracle."""
    from jitllm_amd import _lib as L, synthetic
    from jitllm_amd.projections import QuantizedBatchProjections
    say("mixed types, their runs", rows)
    n, dq, dkv = 2048, 1024, 256
    rq, rk = synthetic.weight(O.Q4_K, dq, n, seed=9930), synthetic.weight(O.Q4_K, dkv, n, seed=9931)
    rv = synthetic.weight(O.Q6_K, dkv, n, seed=9932)
    wq, wk, wv = ctx.load_weight(O.Q4_K, rq, dq, n), ctx.load_weight(O.Q4_K, rk, dkv, n), ctx.load_weight(O.Q6_K, rv, dkv, n)
    X = synthetic.activations((rows, n), seed=9933)
    dx = ctx.from_numpy(X)
    width = dq + 2 * dkv
    proj = QuantizedBatchProjections(ctx, rows, n, width)
    one, two = ctx.float_array(rows * width, fill=UNTOUCHED), ctx.float_array(rows * width, fill=UNTOUCHED)
    proj.fusedQKV(dx, one, wq, wk, wv)
    proj._gemm([wq, wk], dx, two, rows, width, 0, L.JL_STORE)
    proj._gemm([wv], dx, two, rows, width, dq + dkv, L.JL_STORE)
    ctx.sync()
    a, b = one.get().reshape(rows, width), two.get().reshape(rows, width)
    assert np.array_equal(a.view(np.uint32), b.view(np.uint32))
    for cols, t, raw, d in ((slice(0, dq), O.Q4_K, rq, dq), (slice(dq, dq + dkv), O.Q4_K, rk, dkv),
                            (slice(dq + dkv, width), O.Q6_K, rv, dkv)):
        assert rel_err(a[:, cols], O.matmul_batch(t, raw, X, d, n), magnitude(t, raw, X, d, n)) < F16_BOUND
    for w in (wq, wk, wv):
        w.free()
    proj.workspace.free()
