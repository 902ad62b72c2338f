"""Pins the CPU oracle before anything is compared with it (no GPU needed)."""
import numpy as np
import pytest

import fixtures as FX
import np_models as NP
from oracle import pyoracle as O

TYPES = [O.Q8_0, O.Q4_0, O.Q4_K]


def bits(a):
    return np.asarray(a, dtype=np.float32).view(np.uint32)


def assert_bit_equal(a, b):
    a, b = np.asarray(a, np.float32), np.asarray(b, np.float32)
    nan = np.isnan(a)
    assert np.array_equal(nan, np.isnan(b))
    assert np.array_equal(bits(a)[~nan], bits(b)[~nan])


# ---- java.util.Random and String.hashCode: published values -------------------------------

def test_java_random_known_values():
    assert O.JavaRandom(0).next_int() == -1155484576
    assert O.JavaRandom(42).next_int() == -1170105035
    assert O.JavaRandom(0).next_gaussian() == 0.8025330637390305
    r = O.JavaRandom(42)
    assert [r.next_int(10) for _ in range(5)] == [0, 3, 8, 4, 0]
    assert O.java_string_hash("hello") == 99162322
    assert O.java_string_hash("") == 0


def _py_next(seed, nbits):
    seed = (seed * 0x5DEECE66D + 0xB) & ((1 << 48) - 1)
    v = seed >> (48 - nbits)
    if v >= 1 << (nbits - 1) and nbits == 32:
        v -= 1 << 32
    return seed, v


def test_java_random_next_bytes_against_pure_python():
    seed = (20260908 ^ 0x5DEECE66D) & ((1 << 48) - 1)
    want = []
    while len(want) < 37:
        seed, v = _py_next(seed, 32)
        for _ in range(4):
            want.append(v & 0xFF)
            v >>= 8
    got = O.JavaRandom(20260908).next_bytes(37)
    assert list(got) == want[:37]


# ---- fp16 conversions --------------------------------------------------------------------

def test_f16_to_f32_all_patterns():
    allbits = np.arange(65536, dtype=np.uint16)
    want = allbits.view(np.float16).astype(np.float32)
    got = np.array([O.f16_to_f32(int(b)) for b in allbits], dtype=np.float32)
    assert_bit_equal(got, want)
    assert O.f16_to_f32(0x4000) == 2.0
    assert O.f16_to_f32(0x0001) == np.float32(2.0 ** -24)
    assert O.f16_to_f32(0xFBFF) == -65504.0


def test_f32_to_f16_round_to_nearest_even():
    rng = np.random.default_rng(1)
    vals = np.concatenate([
        rng.standard_normal(20000).astype(np.float32) * np.float32(10.0) ** rng.integers(-9, 6, 20000),
        np.array([0.0, -0.0, 65504.0, 65519.99, 65520.0, 1e9, 2.0 ** -24, 2.0 ** -25,
                  2.0 ** -25 * 1.0001, 2.0 ** -14, 6.1e-5, np.inf, -np.inf], dtype=np.float32),
        np.arange(65536, dtype=np.uint16).view(np.float16).astype(np.float32)[:0x7C00],
    ]).astype(np.float32)
    with np.errstate(over="ignore"):
        want = vals.astype(np.float16).view(np.uint16)
    got = np.array([O.f32_to_f16(v) for v in vals], dtype=np.uint16)
    assert np.array_equal(got, want)


# ---- element decode: known answers, closed forms, second wording ---------------------------

def test_q4_0_spec_known_answers():
    """T/backend/tornado/kernels/Q4_0DecodeTest.java:95-126."""
    raw = np.zeros(18, dtype=np.uint8)
    raw[0], raw[1], raw[2], raw[3] = 0x00, 0x40, 0x0F, 0x80
    for alt in (False, True):
        assert O.get_float(O.Q4_0, raw, 0, alt) == 14.0
        assert O.get_float(O.Q4_0, raw, 16, alt) == -16.0
        assert O.get_float(O.Q4_0, raw, 1, alt) == -16.0
        assert O.get_float(O.Q4_0, raw, 17, alt) == 0.0


def test_q8_0_closed_form_all_scales_all_quants():
    """q * d is one correctly rounded product of exact operands: any IEEE float32 multiply agrees."""
    scales = np.arange(65536, dtype=np.uint16)
    raw = np.zeros((65536, 8, 34), dtype=np.uint8)
    raw[:, :, 0] = (scales & 0xFF)[:, None]
    raw[:, :, 1] = (scales >> 8)[:, None]
    raw[:, :, 2:] = np.arange(256, dtype=np.uint8).reshape(8, 32)[None]
    got = O.dequant(O.Q8_0, raw.reshape(-1)).reshape(65536, 256)
    d = scales.view(np.float16).astype(np.float64)
    q = np.arange(256, dtype=np.uint8).view(np.int8).astype(np.float64)
    with np.errstate(invalid="ignore", over="ignore"):
        want = (d[:, None] * q[None, :]).astype(np.float32)
    assert_bit_equal(got, want)


def test_q4_0_closed_form_all_scales_all_nibbles():
    scales = np.arange(65536, dtype=np.uint16)
    raw = np.zeros((65536, 18), dtype=np.uint8)
    raw[:, 0] = scales & 0xFF
    raw[:, 1] = scales >> 8
    # byte i: low nibble i, high nibble 15 - i -> element i has q = i, element 16 + i has q = 15 - i
    raw[:, 2:] = (np.arange(16) | ((15 - np.arange(16)) << 4)).astype(np.uint8)[None]
    got = O.dequant(O.Q4_0, raw.reshape(-1)).reshape(65536, 32)
    d = scales.view(np.float16).astype(np.float64)
    q = np.concatenate([np.arange(16), 15 - np.arange(16)]).astype(np.float64) - 8
    with np.errstate(invalid="ignore", over="ignore"):
        want = (d[:, None] * q[None, :]).astype(np.float32)
    assert_bit_equal(got, want)


@pytest.mark.parametrize("t,seed,blocks", [(O.Q4_0, 20260908, 16), (O.Q4_K, 20260904, 8),
                                            (O.Q8_0, 20260908, 16)])
def test_random_bytes_decode_three_ways(t, seed, blocks):
    """Q4_0DecodeTest.java:36-85 / Q4_KDecodeTest.java:32-75: host wording == device wording, and
    both == the independent numpy statement of the ggml layout."""
    raw = FX.random_bytes(seed, blocks * O.block_bytes(t))
    main = O.dequant(t, raw)
    assert_bit_equal(main, O.dequant_alt(t, raw))
    assert_bit_equal(main, NP.DEQUANT[t](raw))


@pytest.mark.parametrize("t", TYPES)
def test_adversarial_blocks_decode_three_ways(t):
    """QuantizedDeviceDecodeParityTest.java:98-121,191,313,349 (24 blocks, special fp16 scales)."""
    seed = 20260908 + O.java_string_hash(FX.TYPE_NAMES[t])
    raw = FX.adversarial_blocks(t, 24, seed)
    main = O.dequant(t, raw)
    assert_bit_equal(main, O.dequant_alt(t, raw))
    assert_bit_equal(main, NP.DEQUANT[t](raw))


def test_q4_k_scale_unpacking_round_trip():
    """Every (scale, min) in 0..63 survives pack -> the oracle's unpack, at every sub-block."""
    from jitllm_amd import synthetic
    sc = np.arange(64, dtype=np.uint8)
    for j in range(8):
        for mval in (0, 21, 63):
            s = np.zeros((64, 8), dtype=np.uint8)
            m = np.zeros((64, 8), dtype=np.uint8)
            s[:, j] = sc
            m[:, j] = mval
            raw = np.zeros((64, 144), dtype=np.uint8)
            raw[:, 0:2] = np.array([0x00, 0x3C], dtype=np.uint8)  # d = 1
            raw[:, 2:4] = np.array([0x00, 0x3C], dtype=np.uint8)  # dmin = 1
            raw[:, 4:16] = synthetic.pack_q4_k_scales(s, m)
            raw[:, 16:] = 0x11  # every nibble q = 1
            out = O.dequant(O.Q4_K, raw.reshape(-1)).reshape(64, 8, 32)
            assert np.array_equal(out[:, j, 0], sc.astype(np.float32) - mval)
            other = [k for k in range(8) if k != j]
            assert np.all(out[:, other, :] == 0.0)


# ---- Q6_K -----------------------------------------------------------------------------------

def test_q6_k_decode_three_ways():
    """Host wording (Q6_KFloatTensor.java:66-122) == device wording
    (TransformerComputeKernelsQ6_K.java:195-232) == an independent numpy statement of ggml's
    dequantize_row_q6_K, on arbitrary bytes and on blocks with special fp16 scales."""
    raw = FX.random_bytes(20260914, 12 * 210)
    main = O.dequant(O.Q6_K, raw)
    assert_bit_equal(main, O.dequant_alt(O.Q6_K, raw))
    assert_bit_equal(main, NP.DEQUANT[O.Q6_K](raw))
    adv = FX.adversarial_blocks(O.Q6_K, 24, 20260908 + O.java_string_hash("Q6_K"))
    main = O.dequant(O.Q6_K, adv)
    assert_bit_equal(main, O.dequant_alt(O.Q6_K, adv))
    assert_bit_equal(main, NP.DEQUANT[O.Q6_K](adv))


def test_q6_k_layout_known_answers():
    """Where each bit of a super-block lands, written out from the format's description rather
    than from any decoder: byte p of ql plane 0 / 1 of half h holds element 128 h + p (+ 32) in
    its low nibble and 128 h + 64 + p (+ 32) in its high nibble; qh byte p of half h holds bits
    4-5 of elements 128 h + p + 32 g in bit pair g; scale byte 8 h + 2 g + p // 16 applies."""
    def block(d_bits=0x3C00):               # d = 1.0, all scales 1, every q = 0 -> w = -32
        b = np.zeros(210, dtype=np.uint8)
        b[192:208] = 1
        b[208], b[209] = d_bits & 0xFF, d_bits >> 8
        return b
    base = O.dequant(O.Q6_K, block())
    assert np.all(base == -32.0)
    cases = []
    for h in (0, 1):
        for p in (0, 5, 17, 31):
            cases += [(64 * h + p, 0x07, 128 * h + p, 7), (64 * h + p, 0x70, 128 * h + 64 + p, 7),
                      (64 * h + 32 + p, 0x0B, 128 * h + 32 + p, 11), (64 * h + 32 + p, 0xB0, 128 * h + 96 + p, 11)]
            for g in range(4):
                cases.append((128 + 32 * h + p, 2 << (2 * g), 128 * h + 32 * g + p, 32))
    for byte, value, element, q in cases:
        b = block()
        b[byte] = value
        out = O.dequant(O.Q6_K, b)
        want = base.copy()
        want[element] = q - 32
        assert np.array_equal(out, want), (byte, value, element)
    # scales: signed bytes, one per 16 elements in the order half, group, l // 16
    b = block()
    b[192:208] = np.arange(-8, 8, dtype=np.int8).view(np.uint8)
    out = O.dequant(O.Q6_K, b).reshape(2, 4, 2, 16)
    for h in range(2):
        for g in range(4):
            for half16 in range(2):
                sc = -8 + 8 * h + 2 * g + half16
                assert np.all(out[h, g, half16] == np.float32(sc) * np.float32(-32))
    # d is applied first: (d * sc) rounded, then times q
    b = block(0x3555)                                     # d = 0.33325195
    b[192:208] = 3
    b[0] = 0x0F                                           # element 0: q = 15
    d = NP.half_bits_to_f32(np.array([0x3555], dtype=np.uint16))[0]
    want = np.float32(np.float32(d * np.float32(3)) * np.float32(15 - 32))
    assert O.dequant(O.Q6_K, b)[0] == want


def test_q5_k_decode_three_ways_and_layout():
    """Host wording (Q5_KFloatTensor.java:78-122) == device wording
    (TransformerComputeKernelsQ5_K.java:144-220) == an independent numpy statement of ggml's
    dequantize_row_q5_K; and the fifth bit's place written out from the format: bit j of qh[pos]
    belongs to element 32 j + pos (sub-block j), worth 16."""
    for raw in (FX.random_bytes(20260913, 10 * 176),
                FX.adversarial_blocks(O.Q5_K, 24, 20260908 + O.java_string_hash("Q5_K"))):
        main = O.dequant(O.Q5_K, raw)
        assert_bit_equal(main, O.dequant_alt(O.Q5_K, raw))
        assert_bit_equal(main, NP.DEQUANT[O.Q5_K](raw))
    from jitllm_amd import synthetic
    def block():
        b = np.zeros(176, dtype=np.uint8)
        b[0:2] = [0x00, 0x3C]                                        # d = 1, dmin = 0
        b[4:16] = synthetic.pack_q4_k_scales(np.full(8, 1, np.uint8), np.zeros(8, np.uint8))
        return b
    assert np.all(O.dequant(O.Q5_K, block()) == 0.0)
    for pos in (0, 7, 31):
        for j in range(8):
            b = block()
            b[16 + pos] = 1 << j
            want = np.zeros(256, dtype=np.float32)
            want[32 * j + pos] = 16.0
            assert np.array_equal(O.dequant(O.Q5_K, b), want), (pos, j)
        for pair in range(4):
            b = block()
            b[48 + 32 * pair + pos] = 0x93                           # low nibble 3, high nibble 9
            want = np.zeros(256, dtype=np.float32)
            want[64 * pair + pos], want[64 * pair + 32 + pos] = 3.0, 9.0
            assert np.array_equal(O.dequant(O.Q5_K, b), want), (pos, pair)
    # the minimum is subtracted after the product: (d sc) q - dmin m
    b = block()
    b[2:4] = [0x00, 0x38]                                            # dmin = 0.5
    b[4:16] = synthetic.pack_q4_k_scales(np.full(8, 3, np.uint8), np.full(8, 5, np.uint8))
    b[48] = 0x02
    assert O.dequant(O.Q5_K, b)[0] == np.float32(3 * 2 - 0.5 * 5)


@pytest.mark.parametrize("t", [O.Q5_K, O.Q6_K])
def test_k_quant_scalar_dot_and_matmul(t):
    """Q6_KFloatTensor.dot / Q5_KFloatTensor.dot are scalarDot: a strictly sequential fp32 sum of
    decoded weight times x, whatever flavour is asked for; rows are independent."""
    from jitllm_amd import synthetic
    d, n = 5, 512
    raw = synthetic.weight(t, d, n, seed=77)
    x = synthetic.activations(n, seed=78)
    w = NP.DEQUANT[t](raw).reshape(d, n)
    want = NP.scalar_dot_rows(w, x)
    for flavour in (O.DOT_SCALAR, O.DOT_VEC256):
        assert_bit_equal(O.matmul(t, raw, x, d, n, flavour=flavour), want)


# ---- Q4_1, Q5_0, IQ4_XS ---------------------------------------------------------------------

NEW_TYPES = [(O.Q4_1, "Q4_1"), (O.Q5_0, "Q5_0"), (O.IQ4_XS, "IQ4_XS")]


@pytest.mark.parametrize("t,name", NEW_TYPES)
def test_minor_types_decode_three_ways(t, name):
    """Host wording (Q4_1FloatTensor.java:73-94, Q5_0FloatTensor.java:61-85, IQ4_XSFloatTensor.java:
    72-100) == device wording (TransformerComputeKernelsQ4_1.java:59-67, ...Q5_0.java:56-70,
    ...IQ4_XS.java:62-96) == an independent numpy statement of ggml's dequantize_row_*; on random
    bytes and on QuantizedDeviceDecodeParityTest's adversarial blocks."""
    bb = O.block_bytes(t)
    for raw in (FX.random_bytes(20260914 + t, 40 * bb),
                FX.adversarial_blocks(t, 24, 20260908 + O.java_string_hash(name))):
        main = O.dequant(t, raw)
        assert_bit_equal(main, O.dequant_alt(t, raw))
        assert_bit_equal(main, NP.DEQUANT[t](raw))


def test_q4_1_known_answers():
    """Q4_1FloatTensorTest.reconstructsScaleTimesNibblePlusMinimum: nibbles i % 16, d = 0.25,
    m = -1.5 -> 0.25 * nibble - 1.5, exact in fp32; element i < 16 in the low nibble of byte i,
    element i >= 16 in the high nibble of byte i - 16.  The nibble is not recentred (Q4_0 would give
    0.25 * (nibble - 8))."""
    b = np.zeros(20, dtype=np.uint8)
    b[0:2] = np.array([0.25], np.float16).view(np.uint8)
    b[2:4] = np.array([-1.5], np.float16).view(np.uint8)
    nib = np.arange(32) % 16
    b[4:20] = nib[:16] | (nib[16:] << 4)
    want = (0.25 * nib - 1.5).astype(np.float32)
    assert np.array_equal(O.dequant(O.Q4_1, b), want)
    # distinct nibbles in the two halves tell the halves apart
    b[4:20] = np.arange(16) | ((15 - np.arange(16)) << 4)
    want = np.concatenate([0.25 * np.arange(16) - 1.5, 0.25 * (15 - np.arange(16)) - 1.5]).astype(np.float32)
    assert np.array_equal(O.dequant(O.Q4_1, b), want)


def test_q5_0_reads_ggmls_layout():
    """QuantizedDeviceDecodeParityTest.q5_0ReadsGgmlsLayout: d = 1, qh = 0xFFFF0000, byte i =
    i | i << 4 -> weight j is j - 16; and a single fifth bit lands on its own element."""
    b = np.zeros(22, dtype=np.uint8)
    b[0:2] = [0x00, 0x3C]
    b[2:6] = [0x00, 0x00, 0xFF, 0xFF]
    b[6:22] = np.arange(16) | (np.arange(16) << 4)
    assert np.array_equal(O.dequant(O.Q5_0, b), (np.arange(32) - 16).astype(np.float32))
    for j in (0, 5, 15, 16, 23, 31):
        b = np.zeros(22, dtype=np.uint8)
        b[0:2] = [0x00, 0x3C]
        b[2 + j // 8] = 1 << (j % 8)
        want = np.full(32, -16.0, dtype=np.float32)
        want[j] = 0.0
        assert np.array_equal(O.dequant(O.Q5_0, b), want), j


def test_iq4_xs_reads_ggmls_layout():
    """QuantizedDeviceDecodeParityTest.iq4_XSReadsGgmlsLayout: d = 1, group g's scale 33 + g, byte i
    of each group i | (15 - i) << 4 -> weight j < 16 of group g is (1 + g) kvalues[j], weight 16 + i
    is (1 + g) kvalues[15 - i]; the table is ggml's published kvalues_iq4nl."""
    kvalues = [-127, -104, -83, -65, -49, -35, -22, -10, 1, 13, 25, 38, 53, 69, 89, 113]
    b = np.zeros(136, dtype=np.uint8)
    b[0:2] = [0x00, 0x3C]
    scales_h = 0
    for g in range(8):
        ls = 33 + g
        b[4 + g // 2] |= (ls & 0xF) << (4 * (g % 2))
        scales_h |= (ls >> 4) << (2 * g)
    b[2], b[3] = scales_h & 0xFF, scales_h >> 8
    for g in range(8):
        b[8 + 16 * g:8 + 16 * g + 16] = np.arange(16) | ((15 - np.arange(16)) << 4)
    want = np.empty(256, dtype=np.float32)
    for j in range(256):
        g, within = divmod(j, 32)
        q = within if within < 16 else 15 - (within - 16)
        want[j] = (1 + g) * kvalues[q]
    got = O.dequant(O.IQ4_XS, b)
    assert np.array_equal(got, want)
    assert np.array_equal(O.dequant_alt(O.IQ4_XS, b), want)
    # a negative group scale: ls = 0 -> d * -32
    b[2:8] = 0
    assert np.array_equal(O.dequant(O.IQ4_XS, b)[:16], np.float32(-32) * np.array(kvalues, np.float32))


@pytest.mark.parametrize("width", [128, 256])
def test_q4_1_vector_dot_lane_model(width):
    """Q4_1FloatTensor.vectorDot (:105-192): per-lane accumulators against an independent numpy
    model; the lane fold held to a few ulp of the magnitude sum."""
    from jitllm_amd import synthetic
    n = 2048
    raw = synthetic.weight(O.Q4_1, 4, n, seed=21)
    x = synthetic.activations(n, seed=22)
    rb = 20 * n // 32
    for r in range(4):
        row = raw[r * rb:(r + 1) * rb]
        val = NP.vector_lane_values(O.Q4_1, row, x, width)
        want_seq = np.float32(0)
        for v in val:
            want_seq = np.float32(want_seq + v)
        got = O.dot(O.Q4_1, width, raw, r * n, x, 0, n)
        deq = NP.DEQUANT[O.Q4_1](row)
        # the affine form sums d * q * x and m * x apart: the magnitude that bounds its rounding
        mag = np.abs(deq * x).sum() + np.abs(x).sum() * 0.3
        assert abs(float(got) - float(want_seq)) <= 4 * np.finfo(np.float32).eps * mag
        exact = (deq.astype(np.float64) * x).sum()
        assert abs(float(got) - exact) <= 64 * np.finfo(np.float32).eps * mag


def test_q4_1_vector_dot_agrees_with_elementwise_on_spans():
    """Q4_1FloatTensorTest.vectorizedDotAgreesWithElementwise: five blocks, spans {0, size},
    {32, 96}, {0, 100}, {64, 33} (whole, aligned inner, scalar tail, one block + one element), tolerance
    max(1e-4, |expected| * 1e-5) against the float64 elementwise sum."""
    rng = O.JavaRandom(4242)
    blocks, size = 5, 160
    nibbles = np.array([rng.next_int(16) for _ in range(size)])
    raw = np.zeros(blocks * 20, dtype=np.uint8)
    for b in range(blocks):
        scale = np.float32(0.05) + np.float32(rng.next_float()) * np.float32(0.2)
        mn = np.float32(rng.next_float()) - np.float32(0.5)
        raw[20 * b:20 * b + 2] = np.array([scale], np.float16).view(np.uint8)
        raw[20 * b + 2:20 * b + 4] = np.array([mn], np.float16).view(np.uint8)
        nb = nibbles[32 * b:32 * b + 32]
        raw[20 * b + 4:20 * b + 20] = nb[:16] | (nb[16:] << 4)
    x = np.array([rng.next_gaussian() for _ in range(size)]).astype(np.float32)
    deq = NP.DEQUANT[O.Q4_1](raw).astype(np.float64)
    for offset, length in ((0, size), (32, 96), (0, 100), (64, 33)):
        expected = float((deq[offset:offset + length] * x[offset:offset + length]).sum())
        for flavour in (O.DOT_VEC128, O.DOT_VEC256, O.DOT_SCALAR):
            got = float(O.dot(O.Q4_1, flavour, raw, offset, x, offset, length))
            assert abs(got - np.float32(expected)) <= max(1e-4, abs(np.float32(expected)) * 1e-5), (offset, length)


@pytest.mark.parametrize("t", [O.Q5_0, O.IQ4_XS])
def test_block_sum_dots(t):
    """Q5_0FloatTensor.dot (:87-112) sums a block's 32 products on their own and adds the sum to the
    result, IQ4_XSFloatTensor.dot (:102-126) a group's 32; whatever flavour is asked for.  A span
    that starts or ends inside a block goes through scalarDot there."""
    from jitllm_amd import synthetic
    d, n = 5, 1024
    raw = synthetic.weight(t, d, n, seed=79)
    x = synthetic.activations(n, seed=80)
    w = NP.DEQUANT[t](raw).reshape(d, n)
    want = NP.block_sum_dot_rows(w, x)
    for flavour in (O.DOT_SCALAR, O.DOT_VEC256):
        assert_bit_equal(O.matmul(t, raw, x, d, n, flavour=flavour), want)
    # sequential and block-wise sums differ in the last bits: the form is visible
    assert not np.array_equal(want, NP.scalar_dot_rows(w, x))
    be = O.block_elems(t)
    off, length = be - 5, 5 + be + 3          # 5 scalar, one whole block, 3 scalar
    head = np.float32(0)
    for j in range(off, off + 5):
        head = np.float32(head + np.float32(w[0, j] * x[j]))
    mid = NP.block_sum_dot_rows(w[0:1, be:2 * be], x[be:2 * be])[0]
    tail = np.float32(0)
    for j in range(2 * be, 2 * be + 3):
        tail = np.float32(tail + np.float32(w[0, j] * x[j]))
    want1 = np.float32(np.float32(np.float32(0) + head) + mid)
    want1 = np.float32(want1 + tail)
    assert O.dot(t, O.DOT_SCALAR, raw, off, x, off, length) == want1


# ---- dot products -------------------------------------------------------------------------

@pytest.mark.parametrize("t,name", [(O.Q4_0, "q4_0"), (O.Q4_K, "q4_K"), (O.Q8_0, "q8_0")])
def test_scalar_dot_is_the_reference_tests_host_sum(t, name):
    """NativeQuantizedKernelAccelTest.java:106-135: expected[row] = sum over col of
    getFloat(row*N+col) * x[col], sequential float32 -- which is also FloatTensor.scalarDot."""
    raw = FX.probe_blocks(t, FX.probe_seed(name))
    x = FX.probe_x()
    got = O.matmul(t, raw, x, FX.D_PROBE, FX.N_PROBE, O.DOT_SCALAR)
    deq = NP.DEQUANT[t](raw).reshape(FX.D_PROBE, FX.N_PROBE)
    want = NP.scalar_dot_rows(deq, x)
    assert_bit_equal(got, want)


@pytest.mark.parametrize("t", [O.Q8_0, O.Q4_0])
@pytest.mark.parametrize("width", [128, 256])
def test_vector_dot_lane_model(t, width):
    """Per-lane accumulators are fully determined; the final lane fold is held to a few ulp of the
    magnitude sum because the JDK leaves reduceLanes' association open."""
    from jitllm_amd import synthetic
    n = 2048
    raw = synthetic.weight(t, 4, n, seed=11)
    x = synthetic.activations(n, seed=12)
    rb = O.block_bytes(t) * n // 32
    for r in range(4):
        row = raw[r * rb:(r + 1) * rb]
        val = NP.vector_lane_values(t, row, x, width)
        want_seq = np.float32(0)
        for v in val:
            want_seq = np.float32(want_seq + v)
        got = O.dot(t, width, raw, r * n, x, 0, n)
        mag = np.abs(NP.DEQUANT[t](row) * x).sum()
        assert abs(float(got) - float(want_seq)) <= 4 * np.finfo(np.float32).eps * mag
        pairwise = val.astype(np.float64).sum()
        assert abs(float(got) - pairwise) <= 8 * np.finfo(np.float32).eps * mag


@pytest.mark.parametrize("t", TYPES)
def test_dot_flavours_agree_to_rounding(t):
    from jitllm_amd import synthetic
    n, d = 1024, 16
    raw = synthetic.weight(t, d, n, seed=5)
    x = synthetic.activations(n, seed=6)
    ref = (NP.DEQUANT[t](raw).reshape(d, n).astype(np.float64) * x).sum(axis=1)
    mag = np.abs(NP.DEQUANT[t](raw).reshape(d, n).astype(np.float64) * x).sum(axis=1)
    for flavour in (O.DOT_SCALAR, O.DOT_VEC128, O.DOT_VEC256):
        got = O.matmul(t, raw, x, d, n, flavour)
        assert np.max(np.abs(got - ref) / mag) < 2e-6


@pytest.mark.parametrize("t", TYPES)
def test_matmul_thread_count_and_batching_are_invisible(t):
    """FloatTensor.java:123-140: rows are independent dots, so the thread count cannot change a
    bit, and the batched form is B single-vector calls."""
    from jitllm_amd import synthetic
    n, d, B = 512, 37, 5
    raw = synthetic.weight(t, d, n, seed=7)
    X = synthetic.activations((B, n), seed=8)
    for flavour in (O.DOT_SCALAR, O.DOT_VEC256):
        one = O.matmul_batch(t, raw, X, d, n, flavour, nthreads=1)
        many = O.matmul_batch(t, raw, X, d, n, flavour, nthreads=4)
        assert_bit_equal(one, many)
        for b in range(B):
            assert_bit_equal(one[b], O.matmul(t, raw, X[b], d, n, flavour, nthreads=3))


def test_vector_dot_unaligned_head_and_tail_use_scalar():
    from jitllm_amd import synthetic
    raw = synthetic.weight(O.Q8_0, 1, 256, seed=3)
    x = synthetic.activations(256, seed=4)
    # offset 32, size 40: one vector block then an 8-element scalar tail
    got = O.dot(O.Q8_0, O.DOT_VEC256, raw, 32, x, 32, 40)
    val = NP.vector_lane_values(O.Q8_0, raw[34:68], x[32:64], 256)
    head = np.float32(0)
    for v in val:
        head = np.float32(head + v)
    tail = np.float32(0)
    deq = NP.dequant_q8_0(raw)
    for j in range(64, 72):
        tail = np.float32(tail + np.float32(deq[j] * x[j]))
    want = np.float32(np.float32(0) + head)
    want = np.float32(want + tail)
    assert abs(float(got) - float(want)) <= 1e-5 * abs(float(want)) + 1e-6


def test_swiglu_form():
    g = np.array([-30.0, -1.5, 0.0, 0.25, 3.0, 40.0], dtype=np.float32)
    u = np.array([2.0, -1.0, 5.0, 4.0, 0.5, 1.0], dtype=np.float32)
    got = O.swiglu(g, u)
    want = (g / (1.0 + np.exp(-g.astype(np.float64))).astype(np.float32)).astype(np.float32) * u
    assert_bit_equal(got, want.astype(np.float32))
    assert got[2] == 0.0 and got[5] == 40.0


# ---- RMS normalisation and argmax -----------------------------------------------------------

def test_rms_scale_closed_forms():
    """Cases whose answer is known without the formula under test: a constant vector c has
    sum x^2 / n = c^2 exactly when c^2 n is exact in fp32; a power-of-two factor on x with eps = 0
    moves the scale by exactly its inverse; and a float64 evaluation bounds a generic vector."""
    n = 2048
    for c, eps in ((1.0, 0.0), (2.0, 0.0), (0.5, 1e-5), (3.0, 1e-6)):
        x = np.full(n, c, dtype=np.float32)
        want = 1.0 / np.sqrt(np.float64(np.float32(np.float32(c * c) + np.float32(eps))))
        assert O.rms_scale(x, eps) == np.float32(want), (c, eps)
    rng = np.random.default_rng(7)
    x = rng.standard_normal(4096).astype(np.float32)
    base = O.rms_scale(x, 0.0)
    for k in (-3, 1, 5):
        assert O.rms_scale(np.ldexp(x, k).astype(np.float32), 0.0) == np.float32(np.ldexp(base, -k))
    for eps in (1e-5, 1e-6):
        exact = 1.0 / np.sqrt(np.mean(x.astype(np.float64) ** 2) + eps)
        assert abs(float(O.rms_scale(x, eps)) - exact) <= 3e-6 * exact
    # eps matters where the vector is small, and is added after the division by n
    tiny = np.full(64, 1e-4, dtype=np.float32)
    assert abs(float(O.rms_scale(tiny, 1e-5)) - 1.0 / np.sqrt(1e-8 + 1e-5)) < 1e-2
    assert abs(float(O.rms_scale(tiny, 0.0)) - 1e4) < 1.0


def test_rmsnorm_is_weight_times_scaled_x():
    rng = np.random.default_rng(8)
    x = rng.standard_normal(1024).astype(np.float32) * 3
    w = rng.uniform(0.5, 1.5, 1024).astype(np.float32)
    out = O.rmsnorm(x, w, 1e-5)
    ss = O.rms_scale(x, 1e-5)
    assert_bit_equal(out, (w * (ss * x).astype(np.float32)).astype(np.float32))
    # with unit weights and no eps the result has unit mean square
    unit = O.rmsnorm(x, np.ones_like(x), 0.0)
    assert abs(np.mean(unit.astype(np.float64) ** 2) - 1.0) < 1e-5


def test_batched_rms_apply_f16_closed_forms():
    """batchedRmsReduceParallel + batchedRmsApplyFP16: answers that do not come from the formula.  A
    row of +-2 has mean square exactly 4, so with eps = 0 the scale is exactly 0.5 and the output
    is the weight itself (negated where x is -2) rounded to fp16; eps dominating a tiny row gives
    1/sqrt(eps); a row scaled by a power of two has its scale divided by it and the same output."""
    n = 1000
    rng = np.random.default_rng(77)
    w = rng.uniform(0.5, 1.5, n).astype(np.float32)
    signs = rng.choice(np.float32([-1.0, 1.0]), n)
    scales, out = O.batched_rms_apply_f16((2.0 * signs)[None, :], w, 0.0)
    assert scales[0] == np.float32(0.5)
    assert np.array_equal(out[0].view(np.uint16), (w * signs).astype(np.float16).view(np.uint16))
    scales, out = O.batched_rms_apply_f16(np.full((1, n), 1e-20, np.float32), w, 0.25)
    assert scales[0] == np.float32(2.0)
    x = rng.standard_normal((3, n)).astype(np.float32)
    s1, o1 = O.batched_rms_apply_f16(x, w, 0.0)
    s2, o2 = O.batched_rms_apply_f16(x * np.float32(8.0), w, 0.0)
    assert np.array_equal(s1, s2 * np.float32(8.0))
    # (w * s/8) * 8x == (w * s) * x exactly: both factors move by a power of two
    assert np.array_equal(o1.view(np.uint16), o2.view(np.uint16))
    # float64 evaluation: the scale to fp32 accuracy, the output to half an fp16 ulp and a little
    want_scale = 1.0 / np.sqrt(np.mean(x.astype(np.float64) ** 2, axis=1))
    assert np.all(np.abs(s1 - want_scale) <= 3e-6 * want_scale)
    want = w.astype(np.float64) * want_scale[:, None] * x
    assert np.all(np.abs(o1.astype(np.float64) - want) <= np.abs(want) * (2.0 ** -11 + 1e-5) + 2.0 ** -25)


def test_batched_rms_apply_f16_summation_order():
    """The order the reference's kernel states, in a second wording: numpy over the 256 work items at
    once (element t + 256 j is step j of work item t), the partial sums folded as the tree
    partial[:s] += partial[s:2s].  A sequential sum, or the products taken right to left, gives
    other bits on some of these 64 x 4096 values."""
    rng = np.random.default_rng(78)
    for n in (4096, 1000):
        x = (rng.standard_normal((64, n)) * 3.0).astype(np.float32)
        w = rng.uniform(0.5, 1.5, n).astype(np.float32)
        eps = np.float32(1e-5)
        scales, out = O.batched_rms_apply_f16(x, w, float(eps))
        pad = (-n) % 256
        for b in range(x.shape[0]):
            steps = np.concatenate([x[b], np.zeros(pad, np.float32)]).reshape(-1, 256)
            p = np.zeros(256, np.float32)
            for j in range(steps.shape[0]):
                p = p + steps[j] * steps[j]
            s = 128
            while s:
                p[:s] = p[:s] + p[s:2 * s]
                s //= 2
            scale = np.float32(1.0) / np.sqrt(np.float32(p[0] / np.float32(n)) + eps)
            assert scale.dtype == np.float32 and scales[b] == scale
            want = ((w * scale) * x[b]).astype(np.float16)
            assert np.array_equal(out[b].view(np.uint16), want.view(np.uint16))
    # and the order matters: the sequential fp32 sum gives another scale on some rows
    sums = np.cumsum(x * x, axis=1, dtype=np.float32)[:, -1]
    seq = np.float32(1.0) / np.sqrt(sums / np.float32(n) + eps)
    assert seq.dtype == np.float32 and np.any(seq != scales)


def test_batched_rms_apply_f16_with_the_pending_residual():
    """batchedRmsReduceFusedResidual: the add is one fp32 operation per element, written back, and
    everything after it is the plain form over the updated rows (numpy does the add here)."""
    rng = np.random.default_rng(79)
    x = rng.standard_normal((5, 1000)).astype(np.float32)
    delta = (rng.standard_normal((5, 1000)) * 0.3).astype(np.float32)
    w = rng.uniform(0.5, 1.5, 1000).astype(np.float32)
    kept = x.copy()
    updated = []
    s1, o1 = O.batched_rms_apply_f16(x, w, 1e-5, delta=delta, updated=updated)
    assert np.array_equal(x, kept)
    assert np.array_equal(updated[0].view(np.uint32), (x + delta).view(np.uint32))
    s2, o2 = O.batched_rms_apply_f16(x + delta, w, 1e-5)
    assert np.array_equal(s1.view(np.uint32), s2.view(np.uint32)) and np.array_equal(o1.view(np.uint16), o2.view(np.uint16))


def test_argmax_first_maximum_and_nan():
    rng = np.random.default_rng(9)
    x = rng.standard_normal(5000).astype(np.float32)
    assert O.argmax(x) == int(np.argmax(x))
    x[[17, 400, 4999]] = 9.0
    assert O.argmax(x) == 17
    assert O.argmax(np.array([-np.inf, -np.inf], dtype=np.float32)) == 0
    assert O.argmax(np.array([np.nan, 5.0, 7.0], dtype=np.float32)) == 0      # nothing beats a NaN
    assert O.argmax(np.array([1.0, np.nan, 7.0, 7.0], dtype=np.float32)) == 2  # a NaN never wins


# ---- int8 activation path -------------------------------------------------------------------

def test_quantize_q8_definition():
    """Int8GemmKernels.java:75-129: d = amax/127, q = round-half-away(x * (127/amax)), zero block
    -> zero scale and zero quants."""
    rng = np.random.default_rng(9)
    x = rng.standard_normal((6, 64)).astype(np.float32)
    x[1, 0:32] = 0.0
    x[2, 32:64] *= 1e-38
    x[3, 5] = 2.5  # amax element maps to exactly +-127
    q, s = O.quantize_q8(x)
    xb = x.reshape(-1, 32)
    amax = np.abs(xb).max(axis=1)
    assert_bit_equal(s.reshape(-1), (amax / np.float32(127.0)).astype(np.float32))
    assert np.all(q.reshape(-1, 32)[amax == 0] == 0)
    nz = amax >= 4e-37
    inv = (np.float32(127.0) / amax[nz]).astype(np.float32)
    v = (xb[nz] * inv[:, None]).astype(np.float32)
    want = np.sign(v) * np.floor(np.abs(v) + np.float32(0.5))
    assert np.array_equal(q.reshape(-1, 32)[nz], np.clip(want, -127, 127).astype(np.int8))
    assert np.abs(q).max() == 127


def test_int8_gemm_matches_fp64_product_of_the_quantised_operands():
    """Qwen35Q8_0Int8ProjectionAccelTest.java:101-172: m=256, n=384, k=320, seeds 21/22; only the
    fp32 accumulation separates the GEMM from the fp64 product; worst/magnitude < 1e-5."""
    m, n, k = 256, 384, 320
    raw = FX.int8_gemm_weights(n, k, 21)
    a = FX.int8_gemm_activations(m, k, 22)
    q, s = O.quantize_q8(a)
    got = O.gemm_int8_block_scaled(O.Q8_0, q, s, raw, n)
    b = raw.reshape(n, k // 32, 34)
    dw = b[:, :, 0:2].copy().view(np.uint16)[:, :, 0].view(np.float16).astype(np.float64)
    wq = b[:, :, 2:].view(np.int8).astype(np.int64)
    dots = np.einsum("mbi,nbi->mnb", q.reshape(m, k // 32, 32).astype(np.int64), wq)
    terms = dots.astype(np.float64) * s.astype(np.float64)[:, None, :] * dw[None, :, :]
    worst = np.max(np.abs(got - terms.sum(axis=2)) / np.abs(terms).sum(axis=2))
    assert worst < 1e-5


# ---- the packed-integer decode path -----------------------------------------------------------

def test_quantize_q8_blocks_known_answers():
    """quantizeActivationQ8Blocks (TransformerComputeKernelsQ4_0.java:287-341).  With max|x| = 127 the
    inverse is exactly 1, so the rounding rule shows: halves go away from zero, the maximum maps to
    +-127, the scale is max|x| / 127 = 1 and the sum is the sum of the quants; a block of zeros has
    zero scale, quants and sum."""
    x = np.zeros(96, dtype=np.float32)
    x[0:8] = [127.0, -127.0, 2.5, -2.5, 2.4999, -2.4999, 0.49, -0.51]
    x[64:96] = np.linspace(-3, 3, 32)
    q, s, m = O.quantize_q8_blocks(x)
    assert list(q[0:8]) == [127, -127, 3, -3, 2, -2, 0, -1]
    assert s[0] == 1.0 and m[0] == int(q[0:32].astype(np.int64).sum())
    assert s[1] == 0.0 and m[1] == 0 and not q[32:64].any()
    assert s[2] == np.float32(np.float32(3.0) / np.float32(127.0)) and abs(int(q[64])) == 127 and abs(int(q[95])) == 127
    # the same definition as the prefill quantiser (Int8GemmKernels.java:75-129) on ordinary data
    rng = np.random.default_rng(31)
    v = (rng.standard_normal((4, 256)) * 3).astype(np.float32)
    q1, s1, m1 = O.quantize_q8_blocks(v)
    q2, s2 = O.quantize_q8(v)
    assert np.array_equal(q1.reshape(4, 256), q2) and np.array_equal(s1.reshape(4, 8), s2)
    assert np.array_equal(m1, q1.reshape(-1, 32).astype(np.int64).sum(axis=1))


def _grid_activation(n, seed):
    """An activation that lies on its own int8 grid: q random in [-127, 127] with +-127 present in
    every block, times a power-of-two block scale -- quantising it loses nothing."""
    rng = np.random.default_rng(seed)
    q = rng.integers(-127, 128, size=(n // 32, 32)).astype(np.int64)
    q[:, 0] = 127 * rng.choice([-1, 1], size=n // 32)
    scale = np.ldexp(1.0, rng.integers(-9, -3, size=n // 32)).astype(np.float32)
    return (q * scale[:, None]).astype(np.float32).reshape(-1), q.reshape(-1), scale


@pytest.mark.parametrize("t", TYPES)
def test_packed_projection_is_exact_on_the_grid(t):
    """If the activation is exactly representable the packed projection computes the true dot
    product: compared with the float64 product of the decoded weights (numpy statement of the
    format) -- a wrong nibble half, a missing -8 or a swapped scale / minimum fails it."""
    from jitllm_amd import synthetic
    d, n = 12, 1024
    raw = synthetic.weight(t, d, n, seed=41)
    x, q, scale = _grid_activation(n, 42)
    qq, ss, mm = O.quantize_q8_blocks(x)
    assert np.array_equal(qq, q) and np.array_equal(ss, scale * np.float32(127) / np.float32(127))
    w = NP.DEQUANT[t](raw).reshape(d, n).astype(np.float64)
    exact = w @ x.astype(np.float64)
    mag = np.abs(w) @ np.abs(x.astype(np.float64))
    got = O.matmul_q8x(t, raw, qq, ss, mm, d, n)
    # Q4_0 / Q4_K subtract 8 sum / min sum after the product: their terms are up to ~3x the magnitude
    assert np.max(np.abs(got - exact) / mag) < 2e-6


@pytest.mark.parametrize("t", TYPES)
def test_packed_projection_numpy_model(t):
    """The three per-block formulas evaluated independently in numpy (int64 dots, float64 scales)
    on an ordinary activation."""
    from jitllm_amd import synthetic
    d, n = 7, 2048
    raw = synthetic.weight(t, d, n, seed=43)
    x = synthetic.activations(n, seed=44) * np.float32(1.7)
    q, s, m = O.quantize_q8_blocks(x)
    got = O.matmul_q8x(t, raw, q, s, m, d, n)
    qi = q.astype(np.int64).reshape(n // 32, 32)
    s64, m64 = s.astype(np.float64), m.astype(np.int64)
    if t == O.Q8_0:
        b = raw.reshape(d, n // 32, 34)
        dw = NP.half_bits_to_f32(b[:, :, 0:2].copy().view(np.uint16)[:, :, 0]).astype(np.float64)
        wq = b[:, :, 2:].view(np.int8).astype(np.int64)
        want = (dw * s64 * (wq * qi).sum(axis=2)).sum(axis=1)
        mag = (np.abs(dw) * s64 * (np.abs(wq) * np.abs(qi)).sum(axis=2)).sum(axis=1)
    elif t == O.Q4_0:
        b = raw.reshape(d, n // 32, 18)
        dw = NP.half_bits_to_f32(b[:, :, 0:2].copy().view(np.uint16)[:, :, 0]).astype(np.float64)
        nib = np.concatenate([b[:, :, 2:] & 0xF, b[:, :, 2:] >> 4], axis=2).astype(np.int64)
        want = (dw * s64 * ((nib * qi).sum(axis=2) - 8 * m64)).sum(axis=1)
        mag = (np.abs(dw) * s64 * ((nib * np.abs(qi)).sum(axis=2) + 8 * np.abs(m64))).sum(axis=1)
    else:
        b = raw.reshape(d, n // 256, 144)
        dd = NP.half_bits_to_f32(b[:, :, 0:2].copy().view(np.uint16)[:, :, 0]).astype(np.float64)
        dmin = NP.half_bits_to_f32(b[:, :, 2:4].copy().view(np.uint16)[:, :, 0]).astype(np.float64)
        sc, mn = NP.q4_k_scales_mins(b[:, :, 4:16])
        qs = b[:, :, 16:].reshape(d, n // 256, 4, 32)
        nib = np.stack([qs & 0xF, qs >> 4], axis=3).reshape(d, n // 256, 8, 32).astype(np.int64)
        qb = qi.reshape(n // 256, 8, 32)
        sb, mb = s64.reshape(n // 256, 8), m64.reshape(n // 256, 8)
        dots = (nib * qb).sum(axis=3)
        want = (dd[:, :, None] * sc * sb * dots - dmin[:, :, None] * mn * sb * mb).sum(axis=(1, 2))
        mag = (np.abs(dd[:, :, None]) * sc * sb * (nib * np.abs(qb)).sum(axis=3)
               + np.abs(dmin[:, :, None]) * mn * sb * np.abs(mb)).sum(axis=(1, 2))
    assert np.max(np.abs(got - want) / mag) < 2e-6


# ---- Q8_0FloatTensor.dotQ8Activation (-Djitllm.quantizeActivation=true) --------------------------

def _q8_0_row(quants, scales_f16):
    """Q8_0 blocks from int8 values [blocks][32] and binary16 scales [blocks]."""
    blocks = np.zeros((len(scales_f16), 34), dtype=np.uint8)
    blocks[:, 0:2] = np.asarray(scales_f16, dtype=np.float16).view(np.uint8).reshape(-1, 2)
    blocks[:, 2:] = np.asarray(quants, dtype=np.int8).view(np.uint8)
    return blocks.reshape(-1)


def test_quantized_activation_dot_is_exact_on_the_grid():
    """Activations that lie on their own int8 grid with a power-of-two step, weights with power-of-two
    scales: every step of dotQ8Activation (Q8_0FloatTensor.java:107-140) is exact, and the result is
    the integer dot product times the scales -- evaluated here with Python integers and fractions."""
    from fractions import Fraction
    rng = np.random.default_rng(71)
    blocks = 6
    wq = rng.integers(-127, 128, size=(blocks, 32))
    w_exp = rng.integers(-8, -2, size=blocks)
    aq = rng.integers(-127, 128, size=(blocks, 32))
    aq[:, 5] = 127 * rng.choice([-1, 1], size=blocks)       # the block maximum fixes the step
    a_exp = rng.integers(-6, 4, size=blocks)
    x = (aq * np.ldexp(1.0, a_exp)[:, None]).astype(np.float32).reshape(-1)
    raw = _q8_0_row(wq, np.ldexp(1.0, w_exp))
    want = sum(Fraction(int((wq[b] * aq[b]).sum())) * Fraction(2) ** int(w_exp[b] + a_exp[b]) for b in range(blocks))
    got = O.dot(O.Q8_0, O.DOT_Q8ACT, raw, 0, x, 0, blocks * 32)
    assert Fraction(float(got)) == want       # (the six terms and their running sums fit 24 bits)
    # an offset into both operands, as matmul passes them: the last four blocks only
    got = O.dot(O.Q8_0, O.DOT_Q8ACT, raw, 64, x, 64, (blocks - 2) * 32)
    want = sum(Fraction(int((wq[b] * aq[b]).sum())) * Fraction(2) ** int(w_exp[b] + a_exp[b]) for b in range(2, blocks))
    assert Fraction(float(got)) == want


def test_quantized_activation_dot_rounding_and_scale():
    """Halves round away from zero; the integers come from the fp32 scale while the sum is multiplied
    by that scale rounded to binary16 (ggml's order, :123-127); a zero block adds nothing."""
    ones = np.ones((1, 32), dtype=np.int64)
    raw = _q8_0_row(ones, [1.0])
    x = np.zeros(32, dtype=np.float32)
    x[0] = 127.0                       # step 1: s = x
    x[1:6] = [2.5, -2.5, 0.49999997, -0.49999997, 126.5]
    # 127 + 3 - 3 + 0 - 0 + 127
    assert O.dot(O.Q8_0, O.DOT_Q8ACT, raw, 0, x, 0, 32) == 254.0
    # a step that is no binary16 number: 1 + 2^-12 rounds to 1, the integers still use 1 + 2^-12
    step = np.float32(1.0) + np.float32(2.0 ** -12)
    x = np.zeros(32, dtype=np.float32)
    x[0] = np.float32(127.0) * step
    x[1] = np.float32(100.4)
    a_inv = np.float32(1.0) / (x[0] / np.float32(127.0))
    q1 = int(np.float32(x[1] * a_inv) + np.float32(0.5))
    assert O.dot(O.Q8_0, O.DOT_Q8ACT, raw, 0, x, 0, 32) == float(127 + q1)      # not (127 + q1) * step
    assert O.dot(O.Q8_0, O.DOT_Q8ACT, raw, 0, np.zeros(32, np.float32), 0, 32) == 0.0
    # a NaN among the activations quantizes to 0 (Java's (int) of NaN) and is no maximum
    x = np.zeros(32, dtype=np.float32)
    x[0], x[1] = 127.0, np.nan
    assert O.dot(O.Q8_0, O.DOT_Q8ACT, raw, 0, x, 0, 32) == 127.0


def test_quantized_activation_matmul_numpy_model():
    """An independent numpy float32 statement on ordinary input, row by row, bit for bit; the result
    is the true product to within the quantization step; the other types read the flavour as scalar."""
    from jitllm_amd import synthetic
    d, n = 9, 1024
    raw = synthetic.weight(O.Q8_0, d, n, seed=72)
    x = synthetic.activations(n, seed=73) * np.float32(2.3)
    got = O.matmul(O.Q8_0, raw, x, d, n, O.DOT_Q8ACT)
    b = raw.reshape(d, n // 32, 34)
    dw = NP.half_bits_to_f32(b[:, :, 0:2].copy().view(np.uint16)[:, :, 0])
    wq = b[:, :, 2:].view(np.int8).astype(np.int64)
    xb = x.reshape(n // 32, 32)
    amax = np.abs(xb).max(axis=1)
    qs = (amax / np.float32(127.0)).astype(np.float32)
    a_scale = qs.astype(np.float16).astype(np.float32)
    a_inv = (np.float32(1.0) / qs).astype(np.float32)
    s = (xb * a_inv[:, None]).astype(np.float32)
    aq = (s + np.copysign(np.float32(0.5), s)).astype(np.float32).astype(np.int64)    # truncation toward zero
    isum = (wq * aq[None, :, :]).sum(axis=2)
    want = np.zeros(d, dtype=np.float32)
    for blk in range(n // 32):
        want = (want + isum[:, blk].astype(np.float32) * (dw[:, blk] * a_scale[blk]).astype(np.float32)).astype(np.float32)
    assert_bit_equal(got, want)
    w = NP.DEQUANT[O.Q8_0](raw).reshape(d, n).astype(np.float64)
    exact, mag = w @ x.astype(np.float64), np.abs(w) @ np.abs(x.astype(np.float64))
    assert np.max(np.abs(got - exact) / mag) < 5e-3
    assert np.max(np.abs(got - exact) / mag) > 1e-6          # it is not the unquantized product
    raw4 = synthetic.weight(O.Q4_0, d, n, seed=74)
    assert_bit_equal(O.matmul(O.Q4_0, raw4, x, d, n, O.DOT_Q8ACT), O.matmul(O.Q4_0, raw4, x, d, n, O.DOT_SCALAR))
