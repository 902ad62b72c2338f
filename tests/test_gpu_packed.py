"""GPU parity of the packed-integer ("dp4a") decode path: the activation quantiser bit for bit, the
projections against the oracle's statement of the reference's packed arithmetic, and the whole
path against the fp32 CPU path inside the reference's own looser envelope for it."""
import numpy as np
import pytest

from gpu_util import magnitude, rel_err, say
from oracle import pyoracle as O

pytestmark = pytest.mark.gpu

TYPES = [O.Q8_0, O.Q4_0, O.Q4_K]
NAMES = {O.Q8_0: "q8_0", O.Q4_0: "q4_0", O.Q4_K: "q4_K"}
POISON = np.float32(-999999.0)


@pytest.fixture(scope="module")
def ctx():
    from jitllm_amd.runtime import Context
    c = Context(0)
    yield c
    c.close()


def packed_projections(ctx, n, **arrays):
    from jitllm_amd.projections import PackedActivation, QuantizedProjections, TornadoWorkspace
    ws = TornadoWorkspace(packedX=PackedActivation(ctx, n), **arrays)
    return QuantizedProjections(ctx, ws, packed=True), ws


def packed_magnitude(t, raw, q, s, d, n):
    """sum over the row of |w| |x~| with x~ = q * scale, the activation the packed path sees (for
    Q4_0 / Q4_K the recentring and minimum terms are of the same order)."""
    xq = (q.astype(np.float32).reshape(-1, 32) * s[:, None]).reshape(-1)
    return 3.0 * magnitude(t, raw, xq, d, n) + 1e-30


@pytest.mark.parametrize("n", [64, 2048, 4096, 14336])
def test_quantizer_bit_exact(ctx, n):
    """quantizeActivationQ8Blocks: quants, scales and sums equal the oracle's, including a block of
    zeros, exact halves, a block of one huge value and a tiny block."""
    from jitllm_amd import synthetic
    say("quantize", n)
    x = synthetic.activations(n, seed=1200 + n) * np.float32(2.0)
    x[0:32] = 0.0
    x[32:40] = [127.0, -127.0, 2.5, -2.5, 1.5, -1.5, 0.5, -0.5]
    x[40:64] = 0.25
    if n > 64:
        x[64:96] = 1e-30
        x[96:128] = 0.0
        x[100] = 3e38
    proj, ws = packed_projections(ctx, n)
    proj.quantize(ctx.from_numpy(x), n)
    ctx.sync()
    q, s, m = ws.packedX.get()
    wq, wsc, wm = O.quantize_q8_blocks(x)
    assert np.array_equal(q, wq) and np.array_equal(s.view(np.uint32), wsc.view(np.uint32)) and np.array_equal(m, wm)


@pytest.mark.parametrize("n", [2048, 4096, 8192])
def test_rms_apply_and_quantize_bit_exact(ctx, n):
    """rmsApplyAndQuantizeActivationQ8Blocks: the normalised vector it writes equals
    CpuOperations.rmsnorm's (same scale, both products rounded) and its quants, scales and sums are
    the quantiser's over exactly that vector -- one launch, the bits of the two separate steps."""
    from jitllm_amd import synthetic
    say("rms + quantize", n)
    x = synthetic.activations(n, seed=1250 + n) * np.float32(3.0)
    w = np.random.default_rng(1251).uniform(0.5, 1.5, n).astype(np.float32)
    xb = ctx.float_array(n, fill=POISON)
    scale = ctx.float_array(1, fill=POISON)
    proj, ws = packed_projections(ctx, n, wrapXb=xb)
    dx = ctx.from_numpy(x)
    proj.rmsScale(dx, n, 1e-5, scale)
    proj.rmsApplyAndQuantize(dx, ctx.from_numpy(w), scale, n)
    ctx.sync()
    ss = scale.get()[0]
    # the device scale may differ from the host's sequential sum in the last bit: the apply is
    # checked with the scale the device used, the scale itself against the oracle's
    assert abs(float(ss) - float(O.rms_scale(x, 1e-5))) <= 2e-6 * float(ss)
    want = (w * (np.float32(ss) * x).astype(np.float32)).astype(np.float32)
    got = xb.get()
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    q, s, m = ws.packedX.get()
    wq, wsc, wm = O.quantize_q8_blocks(want)
    assert np.array_equal(q, wq) and np.array_equal(s.view(np.uint32), wsc.view(np.uint32)) and np.array_equal(m, wm)


@pytest.mark.parametrize("t", TYPES)
@pytest.mark.parametrize("d,n", [(2048, 2048), (512, 2048), (2048, 8192), (4096, 4096), (1000, 4096), (37, 512),
                                 (300, 14336), (8, 64), (128256 // 8, 2048)])
def test_packed_gemv_matches_the_packed_oracle(ctx, t, d, n):
    """Plain and residual projections: the same integer dots, scales applied per block; only the
    order of the float additions differs from the oracle's."""
    from jitllm_amd import synthetic
    if t == O.Q4_K and n % 256:
        pytest.skip("Q4_K rows are whole super-blocks")
    say("packed gemv", NAMES[t], d, n)
    raw = synthetic.weight(t, d, n, seed=1300 + d % 89)
    x = synthetic.activations(n, seed=1301) * np.float32(1.5)
    acc = ctx.from_numpy(np.full(d, 0.75, dtype=np.float32))
    out = ctx.float_array(d, fill=POISON)
    proj, ws = packed_projections(ctx, n, wrapX=acc)
    proj.quantize(ctx.from_numpy(x), n)
    w = ctx.load_weight(t, raw, d, n)
    proj.packedMatvec(out, w, n, d)
    proj.packedMatvec(acc, w, n, d, residual=True)
    ctx.sync()
    q, s, m = O.quantize_q8_blocks(x)
    ref = O.matmul_q8x(t, raw, q, s, m, d, n)
    mag = packed_magnitude(t, raw, q, s, d, n)
    assert rel_err(out.get(), ref, mag) < 2e-6
    assert rel_err(acc.get(), ref.astype(np.float64) + 0.75, mag + 0.75 * 6e-8) < 2e-6


@pytest.mark.parametrize("t", TYPES)
def test_packed_fused_qkv_and_gate_up(ctx, t):
    from jitllm_amd import synthetic
    say("packed fused", NAMES[t])
    n, dq, dkv, ffn = 2048, 2048, 512, 3000
    rq, rk, rv = (synthetic.weight(t, r, n, seed=1400 + i) for i, r in enumerate((dq, dkv, dkv)))
    r1, r3 = synthetic.weight(t, ffn, n, seed=1405), synthetic.weight(t, ffn, n, seed=1406)
    x = synthetic.activations(n, seed=1407)
    hb = ctx.float_array(ffn, fill=POISON)
    proj, ws = packed_projections(ctx, n, wrapHb=hb)
    proj.quantize(ctx.from_numpy(x), n)
    q, k, v = ctx.float_array(dq, fill=POISON), ctx.float_array(dkv, fill=POISON), ctx.float_array(dkv, fill=POISON)
    proj.packedFusedQKV(q, k, v, ctx.load_weight(t, rq, dq, n), ctx.load_weight(t, rk, dkv, n),
                        ctx.load_weight(t, rv, dkv, n))
    proj.packedGateUp(ctx.load_weight(t, r1, ffn, n), ctx.load_weight(t, r3, ffn, n), n, ffn)
    ctx.sync()
    xq, xs, xm = O.quantize_q8_blocks(x)
    for got, raw, rows in ((q, rq, dq), (k, rk, dkv), (v, rv, dkv)):
        ref = O.matmul_q8x(t, raw, xq, xs, xm, rows, n)
        assert rel_err(got.get(), ref, packed_magnitude(t, raw, xq, xs, rows, n)) < 2e-6
    g = O.matmul_q8x(t, r1, xq, xs, xm, ffn, n)
    u = O.matmul_q8x(t, r3, xq, xs, xm, ffn, n)
    ref = O.swiglu(g, u).astype(np.float64)
    mg, mu = packed_magnitude(t, r1, xq, xs, ffn, n), packed_magnitude(t, r3, xq, xs, ffn, n)
    bound = 4e-6 * (mg * np.abs(u) + 1.2 * mu * np.abs(g)) + 1e-7
    assert np.all(np.abs(hb.get().astype(np.float64) - ref) <= bound)


@pytest.mark.parametrize("t", TYPES)
def test_packed_path_inside_the_references_envelope(ctx, t):
    """Against the fp32 CPU path the packed projection is off by the activation's 8-bit rounding:
    held to the relative L2 (5e-2) and cosine (0.9994) of the reference's bounds for this path
    (CpuGpuParity.Q8_0_PACKED_ACTIVATION), and shown to be far outside the 1e-3 bound of the fp32
    entry points on at least one row -- the two modes are not interchangeable."""
    from jitllm_amd import synthetic
    say("packed envelope", NAMES[t])
    d, n = 4096, 4096
    raw = synthetic.weight(t, d, n, seed=1500)
    x = synthetic.activations(n, seed=1501)
    out = ctx.float_array(d, fill=POISON)
    proj, ws = packed_projections(ctx, n)
    proj.quantize(ctx.from_numpy(x), n)
    proj.packedMatvec(out, ctx.load_weight(t, raw, d, n), n, d)
    ctx.sync()
    got = out.get().astype(np.float64)
    ref = O.matmul(t, raw, x, d, n).astype(np.float64)
    rel_l2 = np.linalg.norm(got - ref) / np.linalg.norm(ref)
    cosine = float(got @ ref / (np.linalg.norm(got) * np.linalg.norm(ref)))
    assert rel_l2 < 5e-2 and cosine > 0.9994, (rel_l2, cosine)
    assert rel_l2 > 1e-4


@pytest.mark.parametrize("d,n", [(2048, 2048), (1000, 4096), (512, 8192)])
def test_packed_q8_0_against_the_cpu_paths_own_quantized_activation_dot(ctx, d, n):
    """The reference's CPU path has the same idea behind a switch: Q8_0FloatTensor.dotQ8Activation
    (-Djitllm.quantizeActivation=true, Q8_0FloatTensor.java:86-140) quantizes the activation per block
    of 32 with the same rounding and multiplies integer sums.  It differs from the device path in one
    step -- the activation scale that multiplies the sum is rounded to binary16 there and kept fp32
    here -- so the two agree to 2^-11 of a row's magnitude, an order closer than either is to the fp32
    path."""
    from jitllm_amd import synthetic
    say("packed gemv against the CPU quantized-activation dot", d, n)
    raw = synthetic.weight(O.Q8_0, d, n, seed=1600 + d % 7)
    x = synthetic.activations(n, seed=1601) * np.float32(1.5)
    out = ctx.float_array(d, fill=POISON)
    proj, ws = packed_projections(ctx, n)
    proj.quantize(ctx.from_numpy(x), n)
    w = ctx.load_weight(O.Q8_0, raw, d, n)
    proj.packedMatvec(out, w, n, d)
    ctx.sync()
    got = out.get()
    assert np.all(got != POISON)
    ref = O.matmul(O.Q8_0, raw, x, d, n, O.DOT_Q8ACT)
    mag = magnitude(O.Q8_0, raw, x, d, n)
    close = rel_err(got, ref, mag)
    far = rel_err(got, O.matmul(O.Q8_0, raw, x, d, n, O.DOT_VEC256), mag)
    assert close < 6e-4, close
    assert far > 4 * close, (close, far)
    w.free()


def test_packed_path_refusals(ctx):
    from jitllm_amd import synthetic
    from jitllm_amd._lib import JitllmHipError, UnsupportedProjection
    from jitllm_amd.projections import PackedActivation
    say("packed refusals")
    with pytest.raises(ValueError, match="blocks of 32"):
        PackedActivation(ctx, 48)
    n = 256
    proj, ws = packed_projections(ctx, n)
    proj.quantize(ctx.from_numpy(synthetic.activations(n, seed=1601)), n)
    out = ctx.float_array(8)
    w6 = ctx.load_weight(O.Q6_K, synthetic.weight(O.Q6_K, 8, n, seed=1602), 8, n)
    with pytest.raises(UnsupportedProjection, match="Q6_K"):
        proj.packedMatvec(out, w6, n, 8)
    proj96, ws96 = packed_projections(ctx, 96)
    proj96.quantize(ctx.from_numpy(synthetic.activations(96, seed=1603)), 96)
    w96 = ctx.load_weight(O.Q8_0, synthetic.weight(O.Q8_0, 8, 96, seed=1604), 8, 96)
    with pytest.raises(UnsupportedProjection, match="row length of 96"):
        proj96.packedMatvec(out, w96, 96, 8)
    # five rows of 68 bytes do not end on a 16-byte boundary: the tile kernel would lose the tail
    proj64, ws64 = packed_projections(ctx, 64)
    proj64.quantize(ctx.from_numpy(synthetic.activations(64, seed=1605)), 64)
    w64 = ctx.load_weight(O.Q8_0, synthetic.weight(O.Q8_0, 5, 64, seed=1606), 5, 64)
    with pytest.raises(UnsupportedProjection, match="packed-activation"):
        proj64.packedMatvec(out, w64, 64, 5)
    # a gate/up tile holds a row of each matrix: its longest row is half the plain projection's
    n = 16384
    projL, wsL = packed_projections(ctx, n, wrapHb=ctx.float_array(8))
    projL.quantize(ctx.from_numpy(synthetic.activations(n, seed=1607)), n)
    wL = ctx.load_weight(O.Q8_0, synthetic.weight(O.Q8_0, 8, n, seed=1608), 8, n)
    projL.packedMatvec(out, wL, n, 8)
    with pytest.raises(UnsupportedProjection, match="up to 8192"):
        projL.packedGateUp(wL, wL, n, 8)
    with pytest.raises(JitllmHipError, match="blocks of 32"):
        from jitllm_amd import _lib as L
        L.check(ctx._lib.jl_quantize_q8(ctx.handle, out.ptr, 8, ws.packedX.quants.ptr, ws.packedX.scales.ptr,
                                        ws.packedX.sums.ptr))
