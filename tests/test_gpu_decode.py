"""GPU parity: element decode (bit-exact) and the decode GEMV family, through the C ABI."""
import numpy as np
import pytest

import fixtures as FX
from gpu_util import bits_equal, magnitude, reference_tolerance_ok, rel_err, say
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


def upload(ctx, t, raw, d, n):
    return ctx.load_weight(t, raw, d, n)


# ---- element decode: bit-exact --------------------------------------------------------------

@pytest.mark.parametrize("t,seed,blocks", [(O.Q4_0, 20260908, 16), (O.Q4_K, 20260904, 8),
                                            (O.Q8_0, 20260908, 16)])
def test_decode_random_bytes_bit_exact(ctx, t, seed, blocks):
    """Q4_0DecodeTest / Q4_KDecodeTest inputs: arbitrary bytes, NaN and Inf scales included."""
    say("decode random", NAMES[t])
    raw = FX.random_bytes(seed, blocks * O.block_bytes(t))
    n = O.block_elems(t)
    w = upload(ctx, t, raw, blocks, n)
    assert bits_equal(w.dequantize(), O.dequant(t, raw))


@pytest.mark.parametrize("t", TYPES)
def test_decode_adversarial_blocks_bit_exact(ctx, t):
    """QuantizedDeviceDecodeParityTest.java:98-121: zero, subnormal, unit and extreme scales."""
    say("decode adversarial", NAMES[t])
    raw = FX.adversarial_blocks(t, 24, 20260908 + O.java_string_hash(FX.TYPE_NAMES[t]))
    w = upload(ctx, t, raw, 24, O.block_elems(t))
    assert bits_equal(w.dequantize(), O.dequant(t, raw))


@pytest.mark.parametrize("t", TYPES)
def test_decode_synthetic_weight_bit_exact(ctx, t):
    from jitllm_amd import synthetic
    say("decode synthetic", NAMES[t])
    d, n = 96, 2048
    raw = synthetic.weight(t, d, n, seed=101)
    w = upload(ctx, t, raw, d, n)
    assert bits_equal(w.dequantize(), O.dequant(t, raw))


def test_q4_0_spec_known_answers_on_device(ctx):
    """Q4_0DecodeTest.java:95-126."""
    raw = np.zeros(18, dtype=np.uint8)
    raw[0], raw[1], raw[2], raw[3] = 0x00, 0x40, 0x0F, 0x80
    say("decode q4_0 known answers")
    out = upload(ctx, O.Q4_0, raw, 1, 32).dequantize().reshape(-1)
    assert (out[0], out[16], out[1], out[17]) == (14.0, -16.0, -16.0, 0.0)


# ---- GEMV: the reference's own kernel test ----------------------------------------------------

@pytest.mark.parametrize("t", TYPES)
def test_matvec_reference_probe(ctx, t):
    """NativeQuantizedKernelAccelTest.java:106-172: N = 512, D = 37, every row written, each within
    max(1e-3, 1e-4 |expected|) of the host's sequential sum."""
    from jitllm_amd.projections import QuantizedProjections, TornadoWorkspace
    say("matvec probe", NAMES[t])
    raw = FX.probe_blocks(t, FX.probe_seed(NAMES[t]))
    x = FX.probe_x()
    expected = O.matmul(t, raw, x, FX.D_PROBE, FX.N_PROBE, O.DOT_SCALAR)
    w = upload(ctx, t, raw, FX.D_PROBE, FX.N_PROBE)
    xd = ctx.from_numpy(x)
    out = ctx.float_array(FX.D_PROBE, fill=POISON)
    proj = QuantizedProjections(ctx, TornadoWorkspace(wrapXb=xd))
    proj.matvec(out, w, FX.N_PROBE, FX.D_PROBE)
    ctx.sync()
    got = out.get()
    assert np.all(got != POISON)
    assert np.all(reference_tolerance_ok(got, expected)), np.abs(got - expected).max()


@pytest.mark.parametrize("t", TYPES)
def test_residual_matvec_reference_probe(ctx, t):
    """matrixVectorGenericWithResidual*: wrapX += w . x."""
    from jitllm_amd.projections import QuantizedProjections, TornadoWorkspace
    say("residual probe", NAMES[t])
    raw = FX.probe_blocks(t, FX.probe_seed(NAMES[t]))
    x = FX.probe_x()
    expected = O.matmul(t, raw, x, FX.D_PROBE, FX.N_PROBE, O.DOT_SCALAR)
    base = np.linspace(-3, 3, FX.D_PROBE).astype(np.float32)
    w = upload(ctx, t, raw, FX.D_PROBE, FX.N_PROBE)
    wrap_x = ctx.from_numpy(base)
    proj = QuantizedProjections(ctx, TornadoWorkspace(wrapX=wrap_x))
    proj.residualMatvec(ctx.from_numpy(x), w, FX.N_PROBE, FX.D_PROBE)
    ctx.sync()
    assert np.all(reference_tolerance_ok(wrap_x.get(), base + expected))


# ---- GEMV at the benchmark's shapes -----------------------------------------------------------

SHAPES = [
    (O.Q8_0, 2048, 2048), (O.Q8_0, 512, 2048), (O.Q8_0, 8192, 2048), (O.Q8_0, 2048, 8192),
    (O.Q8_0, 1001, 2048),                      # ragged: rows not a multiple of the tile
    (O.Q4_0, 4096, 4096), (O.Q4_0, 1024, 4096), (O.Q4_0, 2048, 14336), (O.Q4_0, 1792, 4096),
    (O.Q4_K, 4096, 4096), (O.Q4_K, 1024, 4096), (O.Q4_K, 1536, 12288), (O.Q4_K, 3072, 4096),
    (O.Q8_0, 300, 3072), (O.Q4_0, 300, 5120), (O.Q4_K, 130, 1536),   # S not a power of two
    (O.Q8_0, 77, 96), (O.Q4_0, 5, 32), (O.Q4_K, 9, 256), (O.Q8_0, 3, 32768),  # catch-all kernel
    (O.Q8_0, 5, 64), (O.Q8_0, 3, 128), (O.Q4_0, 7, 64), (O.Q4_0, 3, 192),  # bytes that end off a 16-byte boundary
    (O.Q8_0, 8, 64), (O.Q4_0, 4, 64),                                       # ... and the same widths on one
    # rows of more than 8192 columns (workgroups of 1024 threads, four rows to a tile): whole and
    # ragged tiles, a row length that leaves most of a row's lanes idle, the longest row each type takes
    (O.Q8_0, 1026, 14336), (O.Q8_0, 37, 8256), (O.Q8_0, 21, 15360), (O.Q8_0, 64, 16384),
    (O.Q4_0, 131, 16384), (O.Q4_K, 35, 11008), (O.Q4_K, 2, 16384),
]


@pytest.mark.parametrize("t,d,n", SHAPES)
def test_gemv_matches_oracle(ctx, t, d, n):
    from jitllm_amd import synthetic
    from jitllm_amd.projections import QuantizedProjections, TornadoWorkspace
    say("gemv", NAMES[t], d, n)
    raw = synthetic.weight(t, d, n, seed=1000 + d + n)
    x = synthetic.activations(n, seed=2000 + n)
    flavour = O.DOT_SCALAR if t == O.Q4_K else O.DOT_VEC256
    ref = O.matmul(t, raw, x, d, n, flavour)
    w = upload(ctx, t, raw, d, n)
    out = ctx.float_array(d, fill=POISON)
    QuantizedProjections(ctx, TornadoWorkspace()).floatMatvec(ctx.from_numpy(x), out, w, n, d)
    ctx.sync()
    got = out.get()
    assert np.all(got != POISON)
    err = rel_err(got, ref, magnitude(t, raw, x, d, n))
    assert err < 1e-3, err
    assert err < 2e-5, err  # fp32 arithmetic throughout: only the summation order differs


@pytest.mark.parametrize("scale", [1e-20, 1e-6, 1e6, 1e20])
@pytest.mark.parametrize("t", [O.Q8_0, O.Q4_0, O.Q4_K])
def test_gemv_over_activation_magnitudes(ctx, t, scale):
    """The kernels move powers of two between the weights, the sums and the block scales (the 4-bit
    ones multiply nibbles as binary16 subnormals): none of that may cost range or bits for
    activations forty decades apart."""
    from jitllm_amd import synthetic
    from jitllm_amd.projections import QuantizedProjections, TornadoWorkspace
    d, n = 264, 4096
    say("gemv, activations x", scale, NAMES[t])
    raw = synthetic.weight(t, d, n, seed=1800)
    x = (synthetic.activations(n, seed=1801).astype(np.float64) * scale).astype(np.float32)
    ref = O.matmul(t, raw, x, d, n, O.DOT_SCALAR if t == O.Q4_K else O.DOT_VEC256)
    w = upload(ctx, t, raw, d, n)
    out = ctx.float_array(d, fill=POISON)
    QuantizedProjections(ctx, TornadoWorkspace()).floatMatvec(ctx.from_numpy(x), out, w, n, d)
    ctx.sync()
    assert rel_err(out.get(), ref, magnitude(t, raw, x, d, n)) < 2e-5


@pytest.mark.parametrize("n", [768, 1024, 1536, 2048, 2560, 3072, 3584, 4096, 5120, 7168, 8192, 11008, 14336,
                               16384])
@pytest.mark.parametrize("t", [O.Q8_0, O.Q4_0, O.Q4_K])
def test_fixed_geometry_and_general_kernels_give_the_same_bits(ctx, t, n):
    """A weight of whole tiles runs the kernel compiled for its row length (or, for rows that fill
    their slices only in part -- 768, 1536, 2560, 3072, 3584, 5120, 7168, 11008, 14336 columns -- for
    its slice count); the same weight less its last row has a ragged last tile and runs the general
    one.  Same arithmetic in the same order: the rows they share come out bit for bit equal (plain,
    gate/up, fused q|k|v and their RMS-folding forms)."""
    from jitllm_amd import synthetic
    from jitllm_amd.projections import QuantizedProjections, TornadoWorkspace
    d = 272
    say("fixed vs general", NAMES[t], d, n)
    raw = synthetic.weight(t, d, n, seed=1900 + n)
    raw_up = synthetic.weight(t, d, n, seed=1901 + n)
    row_bytes = raw.size // d
    x = ctx.from_numpy(synthetic.activations(n, seed=1902))
    rms = ctx.from_numpy(np.random.default_rng(1903).uniform(0.5, 1.5, n).astype(np.float32))
    outs = []
    for rows in (d, d - 1):
        w = upload(ctx, t, raw[: rows * row_bytes], rows, n)
        w_up = upload(ctx, t, raw_up[: rows * row_bytes], rows, n)
        out = ctx.float_array(rows, fill=POISON)
        hb = ctx.float_array(rows, fill=POISON)
        ws = TornadoWorkspace(wrapXb=x, wrapHb=hb)
        proj = QuantizedProjections(ctx, ws)
        proj.floatMatvec(x, out, w, n, rows)
        if n <= 8192:
            proj.gateUp(w, w_up, n, rows)
        # fused q|k|v: the weight as q, its first 64 rows as k and as v (whole tiles both times; the
        # second pass, with a ragged q, runs the general kernel)
        q, k, v = ctx.float_array(rows, fill=POISON), ctx.float_array(64, fill=POISON), ctx.float_array(64, fill=POISON)
        wk = upload(ctx, t, raw[: 64 * row_bytes], 64, n)
        wv = upload(ctx, t, raw_up[: 64 * row_bytes], 64, n)
        proj.fusedQKV(x, q, k, v, w, wk, wv)
        ctx.sync()
        got = [out.get(), hb.get(), q.get(), k.get(), v.get()]
        if n <= 8192:
            proj.rmsMatvec(x, rms, None, out, w, n, rows, eps=1e-5)
            proj.fullyFusedRmsNormGateUp(x, rms, 1e-5, w, w_up, n, rows)
            proj.fusedRmsNormQKV(x, q, k, v, rms, None, w, wk, wv, eps=1e-5)
            ctx.sync()
            got += [out.get(), hb.get(), q.get(), k.get(), v.get()]
        outs.append(got)
    assert bits_equal(outs[0][0][: d - 1], outs[1][0])
    if n <= 8192:
        assert bits_equal(outs[0][1][: d - 1], outs[1][1])
        assert bits_equal(outs[0][2][: d - 1], outs[1][2])
        assert bits_equal(outs[0][3], outs[1][3]) and bits_equal(outs[0][4], outs[1][4])
        assert bits_equal(outs[0][2], outs[0][0])   # q of the fused call = the plain projection
        # the RMS-folding forms
        assert bits_equal(outs[0][5][: d - 1], outs[1][5])
        assert bits_equal(outs[0][6][: d - 1], outs[1][6])
        assert bits_equal(outs[0][7][: d - 1], outs[1][7])
        assert bits_equal(outs[0][8], outs[1][8]) and bits_equal(outs[0][9], outs[1][9])
        assert bits_equal(outs[0][7], outs[0][5])


def _random_shapes():
    """Seeded row counts and row lengths across every dispatch of the tile kernel: the
    fixed-geometry instances (whole tiles of 2048 / 4096 / 8192 / 16384-column rows), rows that
    fill their slices only in part, ragged last tiles, the 1024-thread workgroups."""
    rng = np.random.default_rng(20260917)
    shapes = []
    for t, step in ((O.Q8_0, 64), (O.Q4_0, 64), (O.Q4_K, 256)):
        for _ in range(14):
            n = int(rng.integers(1, 16384 // step + 1)) * step
            d = int(rng.integers(1, 400))
            shapes.append((t, d, n))
        for n in (2048, 4096, 8192, 12288):
            shapes.append((t, int(rng.integers(1, 40)) * 8, n))   # whole tiles
    for t in (O.Q8_0, O.Q4_0, O.Q4_K):   # (appended: the shapes above keep their seeds)
        for n in (768, 1024, 1536, 3072, 3584, 5120):
            shapes.append((t, int(rng.integers(1, 20)) * 16, n))  # whole tiles of the other row lengths
    return shapes


@pytest.mark.parametrize("t,d,n", _random_shapes())
def test_gemv_and_residual_on_random_shapes(ctx, t, d, n):
    from jitllm_amd import synthetic
    from jitllm_amd.projections import QuantizedProjections, TornadoWorkspace
    say("gemv, random shape", NAMES[t], d, n)
    raw = synthetic.weight(t, d, n, seed=3000 + d + n)
    x = synthetic.activations(n, seed=3100 + n)
    ref = O.matmul(t, raw, x, d, n, O.DOT_SCALAR if t == O.Q4_K else O.DOT_VEC256)
    mag = magnitude(t, raw, x, d, n)
    w = upload(ctx, t, raw, d, n)
    out = ctx.float_array(d, fill=POISON)
    base = synthetic.activations(d, seed=3200)
    acc = ctx.from_numpy(base)
    proj = QuantizedProjections(ctx, TornadoWorkspace(wrapX=acc))
    dx = ctx.from_numpy(x)
    proj.floatMatvec(dx, out, w, n, d)
    proj.residualMatvec(dx, w, n, d)
    ctx.sync()
    got = out.get()
    assert np.all(got != POISON)
    assert rel_err(got, ref, mag) < 2e-5
    assert rel_err(acc.get(), ref.astype(np.float64) + base, mag + np.abs(base) * 6e-8) < 2e-5


@pytest.mark.parametrize("t,d,n", [(O.Q8_0, 130, 14336), (O.Q4_0, 1022, 14336), (O.Q4_K, 67, 12288)])
def test_residual_matvec_on_long_rows(ctx, t, d, n):
    """x += w . hb at the down projection's row lengths (the 1024-thread workgroups), ragged last tile."""
    from jitllm_amd import synthetic
    from jitllm_amd.projections import QuantizedProjections, TornadoWorkspace
    say("residual, long rows", NAMES[t], d, n)
    raw = synthetic.weight(t, d, n, seed=1500 + d)
    x = synthetic.activations(n, seed=1600 + n)
    ref = O.matmul(t, raw, x, d, n, O.DOT_SCALAR if t == O.Q4_K else O.DOT_VEC256)
    mag = magnitude(t, raw, x, d, n)
    w = upload(ctx, t, raw, d, n)
    base = synthetic.activations(d, seed=1700)
    acc = ctx.from_numpy(base)
    QuantizedProjections(ctx, TornadoWorkspace(wrapX=acc)).residualMatvec(ctx.from_numpy(x), w, n, d)
    ctx.sync()
    assert rel_err(acc.get(), ref.astype(np.float64) + base, mag + np.abs(base) * 6e-8) < 2e-5


@pytest.mark.parametrize("t,dq,dkv,n", [(O.Q8_0, 2048, 512, 2048), (O.Q4_0, 4096, 1024, 4096),
                                         (O.Q4_K, 4096, 1024, 4096), (O.Q8_0, 100, 37, 512)])
def test_fused_qkv(ctx, t, dq, dkv, n):
    from jitllm_amd import synthetic
    from jitllm_amd.projections import QuantizedProjections, TornadoWorkspace
    say("qkv", NAMES[t], dq, dkv, n)
    raws = [synthetic.weight(t, d, n, seed=31 + i) for i, d in enumerate((dq, dkv, dkv))]
    x = synthetic.activations(n, seed=41)
    ws = [upload(ctx, t, r, d, n) for r, d in zip(raws, (dq, dkv, dkv))]
    outs = [ctx.float_array(d, fill=POISON) for d in (dq, dkv, dkv)]
    QuantizedProjections(ctx, TornadoWorkspace()).fusedQKV(ctx.from_numpy(x), *outs, *ws)
    ctx.sync()
    for raw, d, out in zip(raws, (dq, dkv, dkv), outs):
        ref = O.matmul(t, raw, x, d, n)
        assert rel_err(out.get(), ref, magnitude(t, raw, x, d, n)) < 2e-5


@pytest.mark.parametrize("t,dims,n", [(O.Q8_0, (276, 1024, 1024), 3008), (O.Q4_0, (198, 242, 242), 6144),
                                       (O.Q4_K, (64, 512, 256), 5120), (O.Q8_0, (8, 1024, 512), 2048),
                                       (O.Q4_K, (12, 40, 2000), 1536)])
def test_fused_qkv_whose_first_weight_is_the_shortest(ctx, t, dims, n):
    """q | k | v with fewer rows in the first weight than in the others, on rows that fill their
    slices only in part (and on ones that fill them): every weight's tiles are read to their own
    end, whatever the first weight's row count; plain and RMS-folding."""
    from jitllm_amd import synthetic
    from jitllm_amd.projections import QuantizedProjections, TornadoWorkspace
    say("qkv, short first weight", NAMES[t], dims, n)
    raws = [synthetic.weight(t, d, n, seed=3300 + i) for i, d in enumerate(dims)]
    x = synthetic.activations(n, seed=3310)
    rw = (1.0 + 0.25 * synthetic.activations(n, seed=3311)).astype(np.float32)
    xn = O.rmsnorm(x, rw, 1e-5)
    ws = [upload(ctx, t, r, d, n) for r, d in zip(raws, dims)]
    plain = [ctx.float_array(d, fill=POISON) for d in dims]
    folded = [ctx.float_array(d, fill=POISON) for d in dims]
    proj = QuantizedProjections(ctx, TornadoWorkspace())
    dx = ctx.from_numpy(x)
    proj.fusedQKV(dx, *plain, *ws)
    proj.fusedRmsNormQKV(dx, *folded, ctx.from_numpy(rw), None, *ws, eps=1e-5)
    ctx.sync()
    for raw, d, a, b in zip(raws, dims, plain, folded):
        assert rel_err(a.get(), O.matmul(t, raw, x, d, n), magnitude(t, raw, x, d, n)) < 2e-5
        assert rel_err(b.get(), O.matmul(t, raw, xn, d, n), magnitude(t, raw, xn, d, n)) < 2e-5


# Rows of 128 slices (5120, 7168, 8192 columns) put one gate row and one up row in a tile, so 272 rows
# and 271 rows are both whole tiles and both run the fixed-geometry instance: the bit comparison of
# fixed and general kernels cannot reach those instances, and they are held to the oracle here.
WIDE_GATE_UP = [(t, d, n) for t in (O.Q8_0, O.Q4_0, O.Q4_K) for n in (5120, 7168, 8192) for d in (272, 271)]


@pytest.mark.parametrize("t,d,n", [(O.Q8_0, 8192, 2048), (O.Q4_0, 14336, 4096),
                                    (O.Q4_K, 12288, 4096), (O.Q4_K, 37, 512)] + WIDE_GATE_UP)
def test_fused_gate_up(ctx, t, d, n):
    """hb = SiLU(w1 . x) * (w3 . x), held against the host's matVec, matVec, swiGLU sequence
    (InferenceCore.java:127-129)."""
    from jitllm_amd import synthetic
    from jitllm_amd.projections import QuantizedProjections, TornadoWorkspace
    say("gate_up", NAMES[t], d, n)
    r1 = synthetic.weight(t, d, n, seed=51)
    r3 = synthetic.weight(t, d, n, seed=52)
    x = synthetic.activations(n, seed=53)
    g = O.matmul(t, r1, x, d, n)
    u = O.matmul(t, r3, x, d, n)
    ref = O.swiglu(g, u)
    hb = ctx.float_array(d, fill=POISON)
    proj = QuantizedProjections(ctx, TornadoWorkspace(wrapXb=ctx.from_numpy(x), wrapHb=hb))
    proj.gateUp(upload(ctx, t, r1, d, n), upload(ctx, t, r3, d, n), n, d)
    ctx.sync()
    got = hb.get()
    # error of a product: relative errors of gate and up add; scale by the magnitudes of both
    mg = magnitude(t, r1, x, d, n)
    mu = magnitude(t, r3, x, d, n)
    bound = 2e-5 * (mg * np.abs(u) + mu * np.abs(g) * 1.2 + 1e-6)
    assert np.all(np.abs(got.astype(np.float64) - ref) <= bound + 1e-6)


# ---- Q6_K, Q5_K, Q4_1, Q5_0, IQ4_XS: decode and the plain single-token projection --------------

KQ = [O.Q5_K, O.Q6_K, O.Q4_1, O.Q5_0, O.IQ4_XS]
KQ_NAMES = FX.TYPE_NAMES


@pytest.mark.parametrize("t", KQ)
def test_k_quant_decode_bit_exact(ctx, t):
    """Arbitrary bytes, special fp16 scales and a synthetic weight: the device decode equals the
    host tensor's getFloat (Q6_K, Q5_K, Q4_1, Q5_0, IQ4_XSFloatTensor) bit for bit."""
    from jitllm_amd import synthetic
    say("decode", KQ_NAMES[t])
    bb, be = O.block_bytes(t), O.block_elems(t)
    for raw, rows in ((FX.random_bytes(20260914, 12 * bb), 12),
                      (FX.adversarial_blocks(t, 24, 20260908 + O.java_string_hash(KQ_NAMES[t])), 24),
                      (synthetic.weight(t, 40, 512, seed=701), 80)):
        w = upload(ctx, t, raw, rows, raw.size // bb // rows * be)
        assert bits_equal(w.dequantize(), O.dequant(t, raw))


@pytest.mark.parametrize("t", [O.Q6_K, O.Q5_K, O.Q4_1, O.Q5_0, O.IQ4_XS])
@pytest.mark.parametrize("d,n,dual", [(4096, 14336, False), (4099, 11008, False), (10001, 4096, False),
                                      (21000, 2048, False), (4800, 8192, False), (803, 3072, False),
                                      (6144, 4096, True), (5001, 4096, True), (10000, 2048, True)])
def test_k_quants_on_the_tile_kernel(ctx, t, d, n, dual):
    """Q6_K, Q5_K, Q4_1 and Q5_0 weights with rows of 2048 columns and more run the tile kernel
    (LDS-DMA ring; slices of 52.5, 44, 40 and 44 bytes read wherever they fall in the row): whole
    and ragged tiles, rows that do not fill their slices, 1024-thread workgroups, plain / residual /
    gate-up."""
    from jitllm_amd import synthetic
    from jitllm_amd.projections import QuantizedProjections, TornadoWorkspace
    say("k-quant tile kernel", KQ_NAMES[t], d, n, dual)
    raw = synthetic.weight(t, d, n, seed=4000 + d)
    x = synthetic.activations(n, seed=4100 + n)
    ref = O.matmul(t, raw, x, d, n)
    mag = magnitude(t, raw, x, d, n)
    w = upload(ctx, t, raw, d, n)
    dx = ctx.from_numpy(x)
    if not dual:
        out = ctx.float_array(d, fill=POISON)
        base = synthetic.activations(d, seed=4200)
        acc = ctx.from_numpy(base)
        proj = QuantizedProjections(ctx, TornadoWorkspace(wrapX=acc))
        proj.floatMatvec(dx, out, w, n, d)
        proj.residualMatvec(dx, w, n, d)
        ctx.sync()
        assert rel_err(out.get(), ref, mag) < 2e-5
        assert rel_err(acc.get(), ref.astype(np.float64) + base, mag + np.abs(base) * 6e-8) < 2e-5
        return
    raw_up = synthetic.weight(t, d, n, seed=4300 + d)
    up = O.matmul(t, raw_up, x, d, n)
    w_up = upload(ctx, t, raw_up, d, n)
    hb = ctx.float_array(d, fill=POISON)
    # (the host mirror fuses gate/up only where the reference does; the library's entry point takes Q6_K)
    from jitllm_amd import _lib as L
    L.check(L.load().jl_gemv_gate_up(ctx.handle, w.handle, w_up.handle, dx.ptr, hb.ptr))
    ctx.sync()
    want = O.swiglu(ref, up)
    got = hb.get()
    assert np.all(got != POISON)
    # SiLU(g) * u moves with both sums: each is held to 2e-5 of its own magnitude
    mu = magnitude(t, raw_up, x, d, n)
    bound = 2e-5 * (mag * np.abs(up) + mu * np.abs(ref) * 1.2 + 1e-6)
    assert np.all(np.abs(got.astype(np.float64) - want) <= bound + 1e-6)


@pytest.mark.parametrize("t", KQ)
@pytest.mark.parametrize("d,n", [(2048, 2048), (32000, 2048), (2048, 8192), (37, 512), (1000, 256), (4, 4096),
                                 (64, 1024)])
def test_k_quant_gemv_matches_oracle(ctx, t, d, n):
    from jitllm_amd import synthetic
    from jitllm_amd.projections import QuantizedProjections, TornadoWorkspace
    say("gemv", KQ_NAMES[t], d, n)
    raw = synthetic.weight(t, d, n, seed=710 + d % 97)
    x = synthetic.activations(n, seed=720)
    ref = O.matmul(t, raw, x, d, n)
    mag = magnitude(t, raw, x, d, n)
    w = upload(ctx, t, raw, d, n)
    out = ctx.float_array(d, fill=POISON)
    acc = ctx.from_numpy(np.full(d, 0.75, dtype=np.float32))
    proj = QuantizedProjections(ctx, TornadoWorkspace(wrapX=acc))
    dx = ctx.from_numpy(x)
    proj.floatMatvec(dx, out, w, n, d)
    proj.residualMatvec(dx, w, n, d)
    ctx.sync()
    assert rel_err(out.get(), ref, mag) < 2e-5
    assert rel_err(acc.get(), ref.astype(np.float64) + 0.75, mag + 0.75 * 6e-8) < 2e-5


@pytest.mark.parametrize("t", KQ)
def test_k_quants_have_no_fused_single_token_kernels(ctx, t):
    """What has no kernel is refused by name; the caller runs the unfused steps
    (QuantizedProjections.java:386-393, 400-480)."""
    from jitllm_amd import synthetic
    from jitllm_amd._lib import UnsupportedProjection
    from jitllm_amd.projections import QuantizedProjections, TornadoWorkspace
    say("unsupported", KQ_NAMES[t])
    d, n = 16, 256
    w = upload(ctx, t, synthetic.weight(t, d, n, seed=731), d, n)
    x = ctx.from_numpy(synthetic.activations(n, seed=732))
    out = ctx.float_array(d, fill=POISON)
    proj = QuantizedProjections(ctx, TornadoWorkspace(wrapXb=x, wrapHb=out, wrapHb2=ctx.float_array(d)))
    with pytest.raises(UnsupportedProjection, match=KQ_NAMES[t]):
        proj.fusedQKV(x, out, out, out, w, w, w)
    assert proj.fusedGateUp(w, w) == (t == O.Q5_K)     # QuantizedProjections.java:386-393
    with pytest.raises(UnsupportedProjection, match=KQ_NAMES[t]):
        proj.rmsMatvec(x, x, None, out, w, n, d, eps=1e-5)
    # ... and gate/up works either way: one launch for Q5_K, else two projections and an
    # element-wise SwiGLU
    proj.gateUp(w, w, n, d)
    ctx.sync()
    ref = O.matmul(t, synthetic.weight(t, d, n, seed=731), synthetic.activations(n, seed=732), d, n)
    assert np.allclose(out.get(), O.swiglu(ref, ref), rtol=1e-4, atol=1e-5)


@pytest.mark.parametrize("t", KQ)
@pytest.mark.parametrize("d,n", [(12288, 4096), (2048, 2048), (37, 512), (300, 8192), (64, 1280)])
def test_k_quant_fused_gate_up(ctx, t, d, n):
    """hb = SiLU(w1 . x) * (w3 . x) in one launch for the remaining types (the reference fuses it for
    Q5_K, QuantizedProjections.java:386-393), held against the host's matVec, matVec, swiGLU."""
    import ctypes as C
    from jitllm_amd import _lib as L, synthetic
    say("gate_up", KQ_NAMES[t], d, n)
    r1 = synthetic.weight(t, d, n, seed=741)
    r3 = synthetic.weight(t, d, n, seed=742)
    x = synthetic.activations(n, seed=743)
    g = O.matmul(t, r1, x, d, n)
    u = O.matmul(t, r3, x, d, n)
    ref = O.swiglu(g, u)
    hb = ctx.float_array(d, fill=POISON)
    w1, w3 = upload(ctx, t, r1, d, n), upload(ctx, t, r3, d, n)
    L.check(L.load().jl_gemv_gate_up(ctx.handle, w1.handle, w3.handle, ctx.from_numpy(x).ptr, hb.ptr))
    ctx.sync()
    got = hb.get()
    mg, mu = magnitude(t, r1, x, d, n), magnitude(t, r3, x, d, n)
    bound = 2e-5 * (mg * np.abs(u) + mu * np.abs(g) * 1.2 + 1e-6)
    assert np.all(np.abs(got.astype(np.float64) - ref) <= bound + 1e-6)
    w1.free()
    w3.free()


# ---- RMS normalisation folded into the projections, argmax -----------------------------------

@pytest.mark.parametrize("n", [512, 2048, 4096, 8192, 16384, 1000])
def test_rms_scale_on_device(ctx, n):
    from jitllm_amd import synthetic
    from jitllm_amd.projections import QuantizedProjections, TornadoWorkspace
    say("rms scale", n)
    x = synthetic.activations(n, seed=600 + n) * np.float32(2.5)
    scale = ctx.float_array(1, fill=POISON)
    QuantizedProjections(ctx, TornadoWorkspace()).rmsScale(ctx.from_numpy(x), n, 1e-5, scale)
    ctx.sync()
    want = float(O.rms_scale(x, 1e-5))
    assert abs(float(scale.get()[0]) - want) <= 2e-6 * want   # parallel sum against the host's sequential one


@pytest.mark.parametrize("t,dq,dkv,n", [(O.Q8_0, 2048, 512, 2048), (O.Q4_0, 4096, 1024, 4096),
                                         (O.Q4_K, 4096, 1024, 4096), (O.Q8_0, 96, 32, 8192),
                                         # rows that fill their slices only in part
                                         (O.Q8_0, 3072, 1024, 3072), (O.Q4_0, 3584, 512, 3584),
                                         (O.Q4_K, 5120, 1024, 5120), (O.Q8_0, 5120, 1024, 5120)])
def test_fused_rms_qkv(ctx, t, dq, dkv, n):
    """q | k | v of rmsnorm(x), held against the host's rmsnorm followed by three matVecs
    (InferenceCore.java:86-91)."""
    from jitllm_amd import synthetic
    from jitllm_amd.projections import QuantizedProjections, TornadoWorkspace
    say("rms qkv", NAMES[t], dq, dkv, n)
    raws = [synthetic.weight(t, d, n, seed=631 + i) for i, d in enumerate((dq, dkv, dkv))]
    x = synthetic.activations(n, seed=641) * np.float32(3.0)
    rw = (1.0 + 0.25 * synthetic.activations(n, seed=642)).astype(np.float32)
    xn = O.rmsnorm(x, rw, 1e-5)
    ws = [upload(ctx, t, r, d, n) for r, d in zip(raws, (dq, dkv, dkv))]
    outs = [ctx.float_array(d, fill=POISON) for d in (dq, dkv, dkv)]
    proj = QuantizedProjections(ctx, TornadoWorkspace())
    dx, drw, scale = ctx.from_numpy(x), ctx.from_numpy(rw), ctx.float_array(1, fill=POISON)
    proj.rmsScale(dx, n, 1e-5, scale)
    proj.fusedRmsNormQKV(dx, *outs, drw, scale, *ws)
    ctx.sync()
    assert np.array_equal(dx.get(), x)   # the normalised activations are never written back
    refs = [O.matmul(t, raw, xn, d, n) for raw, d in zip(raws, (dq, dkv, dkv))]
    for raw, d, out, ref in zip(raws, (dq, dkv, dkv), outs, refs):
        assert rel_err(out.get(), ref, magnitude(t, raw, xn, d, n)) < 2e-5
    # the same with the scale computed inside the kernel
    for out in outs:
        out.init(POISON)
    proj.fusedRmsNormQKV(dx, *outs, drw, None, *ws, eps=1e-5)
    ctx.sync()
    for raw, d, out, ref in zip(raws, (dq, dkv, dkv), outs, refs):
        assert rel_err(out.get(), ref, magnitude(t, raw, xn, d, n)) < 2e-5


@pytest.mark.parametrize("t,d,n", [(O.Q8_0, 8192, 2048), (O.Q4_0, 14336, 4096),
                                    (O.Q4_K, 12288, 4096), (O.Q8_0, 40, 8192), (O.Q4_K, 37, 512),
                                    # rows that fill their slices only in part
                                    (O.Q8_0, 8192, 3072), (O.Q4_0, 4736, 3584), (O.Q4_K, 3456, 5120),
                                    (O.Q8_0, 3456, 5120)] + WIDE_GATE_UP)
def test_fully_fused_rms_gate_up(ctx, t, d, n):
    """hb = SiLU(w1 . xn) * (w3 . xn) with xn = rmsnorm(x), the scale computed inside the kernel:
    against the host's rmsnorm, matVec, matVec, swiGLU (InferenceCore.java:124-129)."""
    from jitllm_amd import synthetic
    from jitllm_amd.projections import QuantizedProjections, TornadoWorkspace
    say("rms gate_up", NAMES[t], d, n)
    r1 = synthetic.weight(t, d, n, seed=651)
    r3 = synthetic.weight(t, d, n, seed=652)
    x = synthetic.activations(n, seed=653) * np.float32(0.2)
    rw = (1.0 + 0.25 * synthetic.activations(n, seed=654)).astype(np.float32)
    xn = O.rmsnorm(x, rw, 1e-5)
    g = O.matmul(t, r1, xn, d, n)
    u = O.matmul(t, r3, xn, d, n)
    ref = O.swiglu(g, u)
    hb = ctx.float_array(d, fill=POISON)
    proj = QuantizedProjections(ctx, TornadoWorkspace(wrapHb=hb))
    proj.fullyFusedRmsNormGateUp(ctx.from_numpy(x), ctx.from_numpy(rw), 1e-5, upload(ctx, t, r1, d, n),
                                 upload(ctx, t, r3, d, n), n, d)
    ctx.sync()
    got = hb.get()
    mg = magnitude(t, r1, xn, d, n)
    mu = magnitude(t, r3, xn, d, n)
    bound = 2e-5 * (mg * np.abs(u) + mu * np.abs(g) * 1.2 + 1e-6)
    assert np.all(np.abs(got.astype(np.float64) - ref) <= bound + 1e-6)


@pytest.mark.parametrize("t,d,n", [(O.Q8_0, 32000, 2048), (O.Q8_0, 9000, 3072), (O.Q4_K, 7000, 5120)])
def test_rms_vocabulary_projection_and_argmax(ctx, t, d, n):
    """Final norm folded into the vocabulary projection, then the greedy token on the device
    (LogitsQ8_0Layer.java:85-110) against rmsnorm, matVec and FloatTensor.argmax on the host."""
    from jitllm_amd import synthetic
    from jitllm_amd.projections import QuantizedProjections, TornadoWorkspace
    say("rms vocabulary + argmax", d, n)
    raw = synthetic.weight(t, d, n, seed=661)
    x = synthetic.activations(n, seed=662)
    rw = (1.0 + 0.25 * synthetic.activations(n, seed=663)).astype(np.float32)
    xn = O.rmsnorm(x, rw, 1e-5)
    ref = O.matmul(t, raw, xn, d, n)
    proj = QuantizedProjections(ctx, TornadoWorkspace())
    dx, drw, scale = ctx.from_numpy(x), ctx.from_numpy(rw), ctx.float_array(1, fill=POISON)
    logits = ctx.float_array(d, fill=POISON)
    token = ctx.raw_buffer(4)
    proj.rmsScale(dx, n, 1e-5, scale)
    proj.rmsMatvec(dx, drw, scale, logits, upload(ctx, t, raw, d, n), n, d)
    proj.argmax(logits, d, token)
    ctx.sync()
    got = logits.get()
    assert rel_err(got, ref, magnitude(t, raw, xn, d, n)) < 2e-5
    assert int(token.download(np.int32, 1)[0]) == O.argmax(got)
    logits.init(POISON)
    proj.rmsMatvec(dx, drw, None, logits, upload(ctx, t, raw, d, n), n, d, eps=1e-5)
    ctx.sync()
    assert rel_err(logits.get(), ref, magnitude(t, raw, xn, d, n)) < 2e-5


# (type, rows, columns): the first four take the projection kernel that keeps its workgroups' best
# logits; then a row count that is not whole tiles, rows shorter than their padded slices, rows in
# several waves, a type with no such form -- those run the projection and the scan, inside the call
PROJECTION_ARGMAX = [(O.Q8_0, 32000, 2048), (O.Q4_0, 20008, 4096), (O.Q4_K, 16384, 2048), (O.Q4_K, 4100, 4096),
                     (O.Q8_0, 1001, 2048), (O.Q8_0, 9000, 3072), (O.Q4_0, 3000, 8192), (O.Q6_K, 5000, 2048)]


@pytest.mark.parametrize("t,d,n", PROJECTION_ARGMAX)
@pytest.mark.parametrize("rms", ["plain", "scale given", "scale in kernel"])
def test_projection_and_argmax_in_one_call(ctx, t, d, n, rms):
    """matvecArgmax against the calls it stands for -- matvec / rmsMatvec, then argmax: the same
    logits bit for bit, the same token, and that token the host's FloatTensor.argmax of the
    logits.  The weight's best row is repeated further down (other tiles, other workgroups), so the
    first of equal maxima has to win across lanes, waves and workgroups."""
    from jitllm_amd import synthetic
    from jitllm_amd.projections import QuantizedProjections, TornadoWorkspace
    say("projection + argmax", t, d, n, rms)
    if rms != "plain" and t == O.Q6_K:
        pytest.skip("the RMS-folding projections take the three main types only")
    raw = synthetic.weight(t, d, n, seed=671).reshape(d, -1).copy()
    x = synthetic.activations(n, seed=672)
    rw = (1.0 + 0.25 * synthetic.activations(n, seed=673)).astype(np.float32)
    proj = QuantizedProjections(ctx, TornadoWorkspace())
    dx, drw, scale = ctx.from_numpy(x), ctx.from_numpy(rw), ctx.float_array(1, fill=POISON)
    proj.rmsScale(dx, n, 1e-5, scale)
    token = ctx.raw_buffer(8)

    def two_calls(w, logits):
        if rms == "plain":
            proj.floatMatvec(dx, logits, w, n, d)
        else:
            proj.rmsMatvec(dx, drw, scale if rms == "scale given" else None, logits, w, n, d, eps=1e-5)
        proj.argmax(logits, d, token)
        ctx.sync()
        return logits.get(), int(token.download(np.int32, 1)[0])

    def one_call(w, logits):
        token.upload(np.array([-7, -7], dtype=np.int32))
        proj.matvecArgmax(dx, logits, w, n, d, token, rmsWeights=None if rms == "plain" else drw,
                          rmsScale=scale if rms == "scale given" else None, eps=1e-5)
        ctx.sync()
        return logits.get(), int(token.download(np.int32, 1)[0])

    first, _ = two_calls(upload(ctx, t, raw.reshape(-1), d, n), ctx.float_array(d, fill=POISON))
    best = O.argmax(first)
    rng = np.random.default_rng(d + n)
    for at in sorted(set(int(i) for i in rng.integers(0, d, 6)) | {d - 1}):
        raw[at] = raw[best]
    w = upload(ctx, t, raw.reshape(-1), d, n)
    want, want_token = two_calls(w, ctx.float_array(d, fill=POISON))
    got, got_token = one_call(w, ctx.float_array(d, fill=POISON))
    assert bits_equal(got, want)
    assert got_token == want_token == O.argmax(want)
    assert np.count_nonzero(want == want[want_token]) >= 2 and want_token == int(np.flatnonzero(want == want.max())[0])


@pytest.mark.parametrize("t,d,n", [(O.Q8_0, 32000, 2048), (O.Q4_K, 4100, 4096)])
def test_projection_argmax_when_no_logit_is_a_number_or_all_are_equal(ctx, t, d, n):
    """FloatTensor.argmax's corners through the one-call form: an activation vector of zeros (every
    logit 0: token 0), one with a NaN (every logit NaN: token 0), and a second call on the same
    context with a smaller weight, which must not see the first call's candidates."""
    from jitllm_amd import synthetic
    from jitllm_amd.projections import QuantizedProjections, TornadoWorkspace
    say("projection + argmax corners", t, d, n)
    raw = synthetic.weight(t, d, n, seed=681)
    w = upload(ctx, t, raw, d, n)
    proj = QuantizedProjections(ctx, TornadoWorkspace())
    token = ctx.raw_buffer(4)
    logits = ctx.float_array(d, fill=POISON)
    x = synthetic.activations(n, seed=682)
    nan = x.copy()
    nan[n // 3] = np.nan
    for v in (np.zeros(n, dtype=np.float32), nan):
        token.upload(np.array([-7], dtype=np.int32))
        proj.matvecArgmax(ctx.from_numpy(v), logits, w, n, d, token)
        ctx.sync()
        assert int(token.download(np.int32, 1)[0]) == O.argmax(logits.get()) == 0
    proj.matvecArgmax(ctx.from_numpy(x), logits, w, n, d, token)
    ctx.sync()
    assert int(token.download(np.int32, 1)[0]) == O.argmax(logits.get())
    small = 264
    ws = upload(ctx, t, raw[: small * (raw.size // d)], small, n)
    few = ctx.float_array(small, fill=POISON)
    proj.matvecArgmax(ctx.from_numpy(x), few, ws, n, small, token)
    ctx.sync()
    assert bits_equal(few.get(), logits.get()[:small])
    assert int(token.download(np.int32, 1)[0]) == O.argmax(few.get())


@pytest.mark.parametrize("n", [1, 5, 1023, 4097, 128256])
def test_argmax_ties_and_edges(ctx, n):
    from jitllm_amd.projections import QuantizedProjections, TornadoWorkspace
    say("argmax", n)
    proj = QuantizedProjections(ctx, TornadoWorkspace())
    token = ctx.raw_buffer(4)
    rng = np.random.default_rng(n)
    cases = [rng.standard_normal(n).astype(np.float32)]
    tied = rng.integers(0, 4, n).astype(np.float32)           # many equal maxima: the first wins
    cases.append(tied)
    cases.append(np.full(n, -np.inf, dtype=np.float32))        # nothing above -inf: index 0
    if n > 2:
        nan_first = cases[0].copy(); nan_first[0] = np.nan     # nothing beats a NaN at index 0
        nan_mid = cases[0].copy(); nan_mid[n // 2] = np.nan    # a NaN elsewhere never wins
        cases += [nan_first, nan_mid]
    for v in cases:
        proj.argmax(ctx.from_numpy(v), n, token)
        ctx.sync()
        assert int(token.download(np.int32, 1)[0]) == O.argmax(v)


@pytest.mark.parametrize("t,d,n", [(O.Q6_K, 1000, 4096), (O.Q5_K, 264, 2048), (O.IQ4_XS, 96, 256), (O.Q8_0, 16, 96)])
def test_unfused_normalisation_in_front_of_a_projection(ctx, t, d, n):
    """Where there is no RMS-folding launch -- the minor types, a row length the folding kernels
    refuse -- the layer runs the reference's unfused steps: rmsScale (reductionOneBlockWithLayer),
    rmsApply (reductionOneBlock2WithLayer: wrapXb = w * (ss * wrapX), two fp32 roundings) and matvec.
    The apply step is held bit for bit to that formula on the device's own scale, the projection to
    the host's rmsnorm + matVec."""
    from jitllm_amd import synthetic
    from jitllm_amd.projections import QuantizedProjections, TornadoWorkspace
    say("unfused rms", KQ_NAMES.get(t, t), d, n)
    raw = synthetic.weight(t, d, n, seed=3400 + d)
    x = synthetic.activations(n, seed=3401) * np.float32(2.0)
    rw = (1.0 + 0.25 * synthetic.activations(n, seed=3402)).astype(np.float32)
    w = upload(ctx, t, raw, d, n)
    ws = TornadoWorkspace(wrapX=ctx.from_numpy(x), wrapXb=ctx.float_array(n + 8, fill=POISON))
    proj = QuantizedProjections(ctx, ws)
    scale, out = ctx.float_array(1, fill=POISON), ctx.float_array(d, fill=POISON)
    proj.rmsScale(ws.wrapX, n, 1e-5, scale)
    proj.rmsApply(ctx.from_numpy(rw), scale, n)
    proj.matvec(out, w, n, d)
    ctx.sync()
    ss = scale.get()[0]
    xb = ws.wrapXb.get()
    assert np.all(xb[n:] == POISON)
    assert bits_equal(xb[:n], rw * (ss * x))
    assert np.array_equal(ws.wrapX.get(), x)
    xn = O.rmsnorm(x, rw, 1e-5)
    assert rel_err(out.get(), O.matmul(t, raw, xn, d, n), magnitude(t, raw, xn, d, n)) < 2e-5


def test_rms_folding_refuses_what_it_has_no_kernel_for(ctx):
    """A row length the tile kernel does not take is refused by name, never normalised some other
    way (the caller then runs the unfused sequence, as the reference does)."""
    from jitllm_amd import synthetic
    from jitllm_amd._lib import UnsupportedProjection
    from jitllm_amd.projections import QuantizedProjections, TornadoWorkspace
    say("rms unsupported")
    t, d, n = O.Q8_0, 16, 96
    w = upload(ctx, t, synthetic.weight(t, d, n, seed=671), d, n)
    x, rw = ctx.from_numpy(synthetic.activations(n, seed=672)), ctx.float_array(n, fill=1.0)
    out = ctx.float_array(d, fill=POISON)
    proj = QuantizedProjections(ctx, TornadoWorkspace(wrapHb=out))
    with pytest.raises(UnsupportedProjection, match="row length of 96"):
        proj.rmsMatvec(x, rw, None, out, w, n, d, eps=1e-5)
    with pytest.raises(UnsupportedProjection, match="row length of 96"):
        proj.fullyFusedRmsNormGateUp(x, rw, 1e-5, w, w, n, d)
    ctx.sync()
    assert np.all(out.get() == POISON)


def test_mixed_gate_up_runs_two_projections_and_swiglu(ctx):
    """QuantizedProjections.gateUp's unfused branch: gate and up of different types."""
    from jitllm_amd import synthetic
    from jitllm_amd.projections import QuantizedProjections, TornadoWorkspace
    say("gate_up mixed")
    d, n = 512, 1024
    r1 = synthetic.weight(O.Q4_K, d, n, seed=61)
    r3 = synthetic.weight(O.Q8_0, d, n, seed=62)
    x = synthetic.activations(n, seed=63)
    ref = O.swiglu(O.matmul(O.Q4_K, r1, x, d, n), O.matmul(O.Q8_0, r3, x, d, n))
    ws = TornadoWorkspace(wrapXb=ctx.from_numpy(x), wrapHb=ctx.float_array(d),
                          wrapHb2=ctx.float_array(d))
    proj = QuantizedProjections(ctx, ws)
    w1, w3 = upload(ctx, O.Q4_K, r1, d, n), upload(ctx, O.Q8_0, r3, d, n)
    assert not proj.fusedGateUp(w1, w3)
    proj.gateUp(w1, w3, n, d)
    ctx.sync()
    assert np.allclose(ws.wrapHb.get(), ref, rtol=1e-4, atol=1e-4)


def test_errors_name_the_cause(ctx):
    """No silent fallback: unsupported combinations and bad shapes raise."""
    import ctypes as C
    from jitllm_amd import _lib as L, synthetic
    say("errors")
    lib = L.load()
    h = C.c_void_p()
    raw = np.zeros(64, dtype=np.uint8)
    st = lib.jl_weight_upload(ctx.handle, 7, raw.ctypes.data, 1, 32, C.byref(h))  # Q5_1: no kernel
    assert st == L.JL_ERR_UNSUPPORTED and b"ggml type 7" in lib.jl_last_error()
    st = lib.jl_weight_upload(ctx.handle, O.Q8_0, raw.ctypes.data, 1, 48, C.byref(h))
    assert st == L.JL_ERR_INVALID and b"whole number" in lib.jl_last_error()
    w8 = upload(ctx, O.Q8_0, synthetic.weight(O.Q8_0, 64, 256, 1), 64, 256)
    w4 = upload(ctx, O.Q4_K, synthetic.weight(O.Q4_K, 64, 256, 2), 64, 256)
    x, o = ctx.float_array(256, 0.0), ctx.float_array(64, 0.0)
    st = lib.jl_gemv_gate_up(ctx.handle, w8.handle, w4.handle, x.ptr, o.ptr)
    assert st == L.JL_ERR_UNSUPPORTED and b"no fused gate/up kernel" in lib.jl_last_error()
    with pytest.raises(L.UnsupportedProjection):
        L.check(lib.jl_gemv_qkv(ctx.handle, w8.handle, w4.handle, w8.handle, x.ptr, o.ptr, o.ptr, o.ptr))
    assert lib.jl_gemv(ctx.handle, w8.handle, x.ptr, o.ptr, L.JL_SWIGLU) == L.JL_ERR_INVALID
    assert lib.jl_gemv(ctx.handle, None, x.ptr, o.ptr, L.JL_STORE) == L.JL_ERR_INVALID


# ---- run-to-run determinism ---------------------------------------------------------------------

@pytest.mark.parametrize("t", TYPES)
def test_results_do_not_change_from_run_to_run(ctx, t):
    """Every output element has one writer and a fixed summation order -- the residual forms use an
    atomic add only to avoid a load, one per element -- so a call repeated on the same inputs gives
    the same bits: plain, residual, fused q|k|v, gate/up, the RMS-folding and the packed forms."""
    from jitllm_amd import synthetic
    from jitllm_amd.projections import PackedActivation, QuantizedProjections, TornadoWorkspace
    say("determinism", NAMES[t])
    n, d, dkv = 4096, 1536, 512
    raws = [synthetic.weight(t, r, n, seed=1700 + i) for i, r in enumerate((d, dkv, dkv, d))]
    wq, wk, wv, w3 = (ctx.load_weight(t, raw, r, n) for raw, r in zip(raws, (d, dkv, dkv, d)))
    x = ctx.from_numpy(synthetic.activations(n, seed=1710))
    rms = ctx.from_numpy(np.random.default_rng(1711).uniform(0.5, 1.5, n).astype(np.float32))

    def run():
        out, q, k, v = (ctx.float_array(r, fill=0.25) for r in (d, d, dkv, dkv))
        hb, acc = ctx.float_array(d, fill=0.25), ctx.from_numpy(np.full(d, 0.75, dtype=np.float32))
        q2, k2, v2, hb2, pout = (ctx.float_array(r, fill=0.25) for r in (d, dkv, dkv, d, d))
        ws = TornadoWorkspace(wrapX=acc, wrapXb=x, wrapHb=hb, packedX=PackedActivation(ctx, n))
        proj = QuantizedProjections(ctx, ws)
        proj.floatMatvec(x, out, wq, n, d)
        proj.residualMatvec(x, wq, n, d)
        proj.fusedQKV(x, q, k, v, wq, wk, wv)
        proj.gateUp(wq, w3, n, d)
        proj.fusedRmsNormQKV(x, q2, k2, v2, rms, None, wq, wk, wv, eps=1e-5)
        rws = TornadoWorkspace(wrapXb=x, wrapHb=hb2)
        QuantizedProjections(ctx, rws).fullyFusedRmsNormGateUp(x, rms, 1e-5, wq, w3, n, d)
        proj.quantize(x, n)
        proj.packedMatvec(pout, wq, n, d)
        ctx.sync()
        return [a.get().view(np.uint32) for a in (out, acc, q, k, v, hb, q2, k2, v2, hb2, pout)]

    first, second = run(), run()
    for a, b in zip(first, second):
        assert np.array_equal(a, b)


@pytest.mark.parametrize("t,d,n", [(O.Q8_0, 512, 17408), (O.Q4_K, 256, 27648), (O.Q4_0, 64, 28672), (O.Q4_K, 6, 32768),
                                   (O.Q8_0, 10, 16512), (O.Q4_0, 1026, 25600), (O.Q4_K, 2048, 25600),
                                   (O.Q8_0, 7, 17408), (O.Q4_0, 4, 16416)])
def test_rows_of_more_than_16384_columns(ctx, t, d, n):
    """The down projections of the largest models (17 408, 25 600, 27 648, 28 672 columns): a thread of
    the tile kernel owns 64 columns and a workgroup has 1 024 threads, so such a row is taken as two
    half rows whose sums meet in the thread that finishes the row.  Plain and residual, against the
    oracle on every output, twice with the same bits; an odd row count and a row length that does not
    halve into whole 64-column slices (the last two cases) go to the catch-all kernel and hold too."""
    from jitllm_amd import synthetic
    from jitllm_amd.projections import QuantizedProjections, TornadoWorkspace
    say("long rows", t, d, n)
    raw = synthetic.weight(t, d, n, seed=9900 + d)
    x = synthetic.activations(n, seed=9901)
    base = synthetic.activations(d, seed=9902)
    w = ctx.load_weight(t, raw, d, n)
    dx = ctx.from_numpy(x)
    ref = O.matmul(t, raw, x, d, n, O.DOT_SCALAR if t == O.Q4_K else O.DOT_VEC256)
    mag = magnitude(t, raw, x, d, n)
    runs = []
    for _ in range(2):
        out = ctx.float_array(d, fill=POISON)
        acc = ctx.from_numpy(base.copy())
        proj = QuantizedProjections(ctx, TornadoWorkspace(wrapX=acc))
        proj.floatMatvec(dx, out, w, n, d)
        proj.residualMatvec(dx, w, n, d)
        ctx.sync()
        runs.append((out.get(), acc.get()))
        out.free()
        acc.free()
    got, added = runs[0]
    assert np.all(got != POISON)
    assert rel_err(got, ref, mag) < 2e-5
    assert rel_err(added - base, ref, mag + np.abs(base) * 1e-6) < 2e-5
    assert bits_equal(got, runs[1][0]) and bits_equal(added, runs[1][1])
    w.free()
