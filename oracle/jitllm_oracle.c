/*
 * jitllm_oracle.c -- CPU restatement of jitLLM's Java CPU quantized matmul.
 *
 * TEST INFRASTRUCTURE ONLY: the checker for the HIP path, never a fallback for it.
 * Built with -ffp-contract=off: Java never contracts a*b+c, so the only fused
 * multiply-adds below are the explicit fmaf() calls that restate FloatVector.fma.
 *
 * J = src/main/java/org/beehive/jitllm in the reference checkout.
 *
 * Pinning (see tests/test_oracle_*.py):
 *   decode (jo_get_float)      known answers of Q4_0DecodeTest, one-rounding closed forms over all
 *                              65536 fp16 scales, agreement with the second wording
 *                              (jo_get_float_alt) on the reference's random and adversarial blocks.
 *   scalar dot                 strictly sequential fp32; brute force against an independent numpy
 *                              float32 loop.
 *   vector dot (128/256)       per-block lane values are fully determined and are compared with an
 *                              independent numpy float32 model; the final reduceLanes(ADD)
 *                              association is NOT specified by the JDK -- lane order 0..7 from
 *                              zero is used here (what the JDK's own fallback does) and the result
 *                              is held to a few ulp, not bit equality: "parity unpinned" for the
 *                              last bits of that one addition chain only.
 *   Q4_1, Q5_0, IQ4_XS         decode: the reference's own known answers (Q4_1FloatTensorTest,
 *                              QuantizedDeviceDecodeParityTest q5_0 / iq4_XS ReadsGgmlsLayout), second
 *                              wordings, numpy statements of ggml's dequantize_row_*; dots: Q4_1 lane
 *                              model as above, Q5_0 / IQ4_XS block sums bit-equal to a numpy loop.
 *   Q8_0 quantized-activation dot (JO_DOT_Q8ACT)  activations on their own int8 grid with power-of-two
 *                              scales make every step exact: the result is the integer dot product
 *                              times the scales, computed with Python integers; halves round away
 *                              from zero; the integer values come from the fp32 scale and the sum
 *                              is multiplied by the binary16-rounded one (a block whose scale is
 *                              not a binary16 number shows the difference); a zero block adds
 *                              nothing; an independent numpy float32 statement on random input.
 *   packed path                quantiser: known answers (the maximum maps to +-127, halves round away
 *                              from zero, a zero block gives zero scale and quants, sums = sum q);
 *                              projections: an activation that lies on its own int8 grid makes the
 *                              packed result the exact dot product, checked against the float64
 *                              product of the decoded weights, and a numpy int64 evaluation of the
 *                              three per-block formulas.
 *   rmsnorm, argmax            closed forms (constant vectors, powers of two, eps-dominated input), a
 *                              float64 evaluation, numpy's argmax with ties, -inf and NaN cases.
 *   batched RMS apply to fp16  closed forms (a row of +-2 returns the weights, eps-dominated rows,
 *                              power-of-two scaling leaves every output bit), a float64 evaluation,
 *                              and the kernel's summation order restated in numpy over the 256 work
 *                              items at once, bit for bit; the residual form against numpy's add.
 *   java.util.Random           published first outputs for seeds 0 and 42.
 */
#include "jitllm_oracle.h"

#include <math.h>
#include <omp.h>
#include <stdlib.h>
#include <string.h>

#define Q_BLOCK 32
#define Q8_0_BYTES 34
#define Q4_0_BYTES 18
#define QK_K 256
#define Q4_K_BYTES 144
#define Q6_K_BYTES 210
#define Q5_K_BYTES 176
#define Q4_1_BYTES 20
#define Q5_0_BYTES 22
#define IQ4_XS_BYTES 136

int jo_max_threads(void) { return omp_get_max_threads(); }

/* J/format/GGMLType.java:7,13,18-20 */
int jo_block_elems(int type) {
    switch (type) {
        case JO_Q4_0: return Q_BLOCK;
        case JO_Q8_0: return Q_BLOCK;
        case JO_Q4_K: return QK_K;
        case JO_Q6_K: return QK_K;
        case JO_Q5_K: return QK_K;
        case JO_Q4_1: return Q_BLOCK;
        case JO_Q5_0: return Q_BLOCK;
        case JO_IQ4_XS: return QK_K;
        default: return 0;
    }
}

int jo_block_bytes(int type) {
    switch (type) {
        case JO_Q4_0: return Q4_0_BYTES;
        case JO_Q8_0: return Q8_0_BYTES;
        case JO_Q4_K: return Q4_K_BYTES;
        case JO_Q6_K: return Q6_K_BYTES;
        case JO_Q5_K: return Q5_K_BYTES;
        case JO_Q4_1: return Q4_1_BYTES;
        case JO_Q5_0: return Q5_0_BYTES;
        case JO_IQ4_XS: return IQ4_XS_BYTES;
        default: return 0;
    }
}

/* ---- Float.float16ToFloat / Float.floatToFloat16 (J/tensor/standard/FloatTensor.java:71-79 call sites) */

static inline float bits_to_float(uint32_t u) {
    float f;
    memcpy(&f, &u, 4);
    return f;
}

static inline uint32_t float_to_bits(float f) {
    uint32_t u;
    memcpy(&u, &f, 4);
    return u;
}

/* IEEE binary16 -> binary32, exact; subnormals widened, NaN payload kept in the top bits. */
float jo_f16_to_f32(uint16_t h) {
    uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1Fu;
    uint32_t man = h & 0x3FFu;
    if (exp == 0) {
        if (man == 0) return bits_to_float(sign);
        /* subnormal: man * 2^-24, exactly representable */
        float v = (float)man * 5.9604644775390625e-8f;
        return bits_to_float(float_to_bits(v) | sign);
    }
    if (exp == 31) return bits_to_float(sign | 0x7F800000u | (man << 13));
    return bits_to_float(sign | ((exp + 112u) << 23) | (man << 13));
}

/* binary32 -> binary16, round to nearest even (Float.floatToFloat16). */
uint16_t jo_f32_to_f16(float value) {
    uint32_t u = float_to_bits(value);
    uint32_t sign = (u >> 16) & 0x8000u;
    uint32_t abs = u & 0x7FFFFFFFu;
    if (abs > 0x7F800000u) return (uint16_t)(sign | 0x7E00u | ((abs >> 13) & 0x1FFu)); /* NaN */
    if (abs >= 0x477FF000u) return (uint16_t)(sign | 0x7C00u); /* >= 65520 rounds to infinity */
    if (abs < 0x33000001u) return (uint16_t)sign;              /* <= 2^-25 rounds to zero */
    int32_t e = (int32_t)(abs >> 23) - 127;
    uint32_t man = (abs & 0x7FFFFFu) | 0x800000u;
    int shift = (e < -14) ? (13 + (-14 - e)) : 13;
    uint32_t half = man >> shift;
    uint32_t rem = man & ((1u << shift) - 1u);
    uint32_t mid = 1u << (shift - 1);
    if (rem > mid || (rem == mid && (half & 1u))) half++;
    if (e < -14) return (uint16_t)(sign | half); /* subnormal; a carry lands on the smallest normal */
    return (uint16_t)(sign | (((uint32_t)(e + 15) << 10) + (half - 0x400u)));
}

static inline uint16_t read_u16(const uint8_t *p) { return (uint16_t)(p[0] | (p[1] << 8)); }

/* ---- element decoders ---------------------------------------------------------------------- */

/* J/tensor/standard/Q8_0FloatTensor.java:52-61 */
static inline float q8_0_get(const uint8_t *w, int64_t index) {
    int64_t block_index = index / Q_BLOCK;
    int64_t within = index % Q_BLOCK;
    const uint8_t *blk = w + block_index * Q8_0_BYTES;
    int8_t quant = (int8_t)blk[2 + within];
    float scale = jo_f16_to_f32(read_u16(blk));
    return (float)quant * scale;
}

/* J/tensor/standard/Q4_0FloatTensor.java:55-79 */
static inline float q4_0_get(const uint8_t *w, int64_t index) {
    int64_t block_index = index / Q_BLOCK;
    const uint8_t *blk = w + block_index * Q4_0_BYTES;
    float scale = jo_f16_to_f32(read_u16(blk));
    int mod = (int)(index % Q_BLOCK);
    int8_t quant;
    if (mod < Q_BLOCK / 2) {
        quant = (int8_t)(blk[2 + mod] & 0x0F);
    } else {
        quant = (int8_t)((blk[2 + mod - Q_BLOCK / 2] >> 4) & 0x0F);
    }
    quant = (int8_t)(quant - 8);
    return (float)quant * scale;
}

/* J/tensor/standard/Q4_KFloatTensor.java:68-75 */
static inline int q4_k_scale(int j, const uint8_t *s) {
    if (j < 4) return s[j] & 63;
    return (s[j + 4] & 0xF) | ((s[j - 4] >> 6) << 4);
}

/* J/tensor/standard/Q4_KFloatTensor.java:78-85 */
static inline int q4_k_min(int j, const uint8_t *s) {
    if (j < 4) return s[j + 4] & 63;
    return (s[j + 4] >> 4) | ((s[j] >> 6) << 4);
}

/* J/tensor/standard/Q4_KFloatTensor.java:87-122 */
static inline float q4_k_get(const uint8_t *w, int64_t index) {
    int64_t block_index = index / QK_K;
    int within = (int)(index % QK_K);
    const uint8_t *blk = w + block_index * Q4_K_BYTES;
    float d = jo_f16_to_f32(read_u16(blk));
    float dmin = jo_f16_to_f32(read_u16(blk + 2));
    const uint8_t *scales = blk + 4;
    int pair = within / 64;
    int pos = within % 64;
    int sub, q;
    if (pos < 32) {
        sub = pair * 2;
        q = blk[16 + pair * 32 + pos] & 0xF;
    } else {
        sub = pair * 2 + 1;
        q = (blk[16 + pair * 32 + (pos - 32)] >> 4) & 0xF;
    }
    int sc = q4_k_scale(sub, scales);
    int m = q4_k_min(sub, scales);
    /* d * sc * q - dmin * m, left to right, every product and the difference rounded to fp32 */
    float t = d * (float)sc;
    t = t * (float)q;
    float u = dmin * (float)m;
    return t - u;
}

/*
 * J/tensor/standard/Q6_KFloatTensor.java:66-122.  A super-block is ql[128] | qh[64] | 16 signed
 * scales | fp16 d; two halves of 128 elements, four groups of 32 in each: the group picks the ql
 * plane (0 / 32), the nibble (low for groups 0-1, high for 2-3) and the bit pair of qh;
 * w = d * scale * (q - 32), left to right in fp32.
 */
static inline float q6_k_get(const uint8_t *w, int64_t index) {
    int64_t block_index = index / QK_K;
    int within = (int)(index % QK_K);
    const uint8_t *blk = w + block_index * Q6_K_BYTES;
    float d = jo_f16_to_f32(read_u16(blk + 208));
    int half_index = within / 128;
    int pos_in_half = within % 128;
    int group = pos_in_half / 32;
    int pos = pos_in_half % 32;
    const uint8_t *ql = blk + half_index * 64;
    const uint8_t *qh = blk + 128 + half_index * 32;
    const int8_t *sc = (const int8_t *)(blk + 192 + half_index * 8);
    int is = pos / 16;
    int q;
    switch (group) {
        case 0: q = ((ql[pos] & 0xF) | (((qh[pos] >> 0) & 3) << 4)) - 32; break;
        case 1: q = ((ql[32 + pos] & 0xF) | (((qh[pos] >> 2) & 3) << 4)) - 32; break;
        case 2: q = ((ql[pos] >> 4) | (((qh[pos] >> 4) & 3) << 4)) - 32; break;
        default: q = ((ql[32 + pos] >> 4) | (((qh[pos] >> 6) & 3) << 4)) - 32; break;
    }
    float t = d * (float)sc[is + 2 * group];
    return t * (float)q;
}

/*
 * J/tensor/standard/Q5_KFloatTensor.java:78-122.  A super-block is fp16 d, dmin | 12 packed scale /
 * min bytes (as Q4_K) | qh[32] | qs[128]: element pos < 32 of pair p is the low nibble of
 * qs[32 p + pos] with bit 2 p of qh[pos] as its fifth bit (sub-block 2 p), element 32 + pos the high
 * nibble with bit 2 p + 1 (sub-block 2 p + 1); w = d * sc * q - dmin * m, left to right in fp32.
 */
static inline float q5_k_get(const uint8_t *w, int64_t index) {
    int64_t block_index = index / QK_K;
    int within = (int)(index % QK_K);
    const uint8_t *blk = w + block_index * Q5_K_BYTES;
    float d = jo_f16_to_f32(read_u16(blk));
    float dmin = jo_f16_to_f32(read_u16(blk + 2));
    const uint8_t *scales = blk + 4;
    int pair = within / 64;
    int pos = within % 64;
    int sub, q, high_bit;
    if (pos < 32) {
        sub = pair * 2;
        q = blk[48 + pair * 32 + pos] & 0xF;
        high_bit = (blk[16 + pos] >> (pair * 2)) & 1;
    } else {
        sub = pair * 2 + 1;
        q = (blk[48 + pair * 32 + (pos - 32)] >> 4) & 0xF;
        high_bit = (blk[16 + (pos - 32)] >> (pair * 2 + 1)) & 1;
    }
    q += high_bit * 16;
    int sc = q4_k_scale(sub, scales);
    int m = q4_k_min(sub, scales);
    float t = d * (float)sc;
    t = t * (float)q;
    float u = dmin * (float)m;
    return t - u;
}

/*
 * J/tensor/standard/Q4_1FloatTensor.java:73-94.  fp16 d | fp16 m | 16 nibble bytes: element i < 16 is
 * the low nibble of byte i, element i >= 16 the high nibble of byte i - 16; w = nibble * d + m,
 * product rounded, then the sum (the nibble is never recentred).
 */
static inline float q4_1_get(const uint8_t *w, int64_t index) {
    const uint8_t *blk = w + (index / Q_BLOCK) * Q4_1_BYTES;
    int within = (int)(index % Q_BLOCK);
    float scale = jo_f16_to_f32(read_u16(blk));
    float min = jo_f16_to_f32(read_u16(blk + 2));
    int nibble = within < 16 ? (blk[4 + within] & 0x0F) : ((blk[4 + within - 16] >> 4) & 0x0F);
    float t = (float)nibble * scale;
    return t + min;
}

/*
 * J/tensor/standard/Q5_0FloatTensor.java:61-85.  fp16 d | 32 fifth bits (little-endian word, bit i
 * belongs to element i) | 16 nibble bytes laid out as Q4_0's; w = d * (q - 16).
 */
static inline float q5_0_decode(const uint8_t *blk, float scale, uint32_t qh, int within) {
    int half = within / 16;
    int packed = blk[6 + within - half * 16];
    int q = ((packed >> (half * 4)) & 0x0F) | (int)(((qh >> within) & 1u) << 4);
    return scale * (float)(q - 16);
}

static inline uint32_t q5_0_high_bits(const uint8_t *blk) {
    return (uint32_t)blk[2] | ((uint32_t)blk[3] << 8) | ((uint32_t)blk[4] << 16) | ((uint32_t)blk[5] << 24);
}

static inline float q5_0_get(const uint8_t *w, int64_t index) {
    const uint8_t *blk = w + (index / Q_BLOCK) * Q5_0_BYTES;
    return q5_0_decode(blk, jo_f16_to_f32(read_u16(blk)), q5_0_high_bits(blk), (int)(index % Q_BLOCK));
}

/*
 * J/tensor/standard/IQ4_XSFloatTensor.java:27-100.  fp16 d | 16 bits scales_h (two high bits of
 * each of the 8 group scales, group g at bit 2 g) | 4 bytes scales_l (low four bits, group g in
 * byte g / 2) | 128 nibble bytes, 16 per group of 32 (elements 0..15 low nibbles, 16..31 high);
 * w = (d * (ls - 32)) * kvalues_iq4nl[nibble].
 */
static const int8_t IQ4NL_VALUES[16] = {-127, -104, -83, -65, -49, -35, -22, -10, 1, 13, 25, 38, 53, 69, 89, 113};

static inline float iq4_xs_group_scale(const uint8_t *blk, float d, int g) {
    int scales_h = read_u16(blk + 2);
    int low = blk[4 + g / 2];
    int ls = ((low >> (4 * (g % 2))) & 0xF) | (((scales_h >> (2 * g)) & 3) << 4);
    return d * (float)(ls - 32);
}

static inline float iq4_xs_decode(const uint8_t *blk, float dl, int g, int within) {
    int half = within / 16;
    int packed = blk[8 + g * 16 + within - half * 16];
    return dl * (float)IQ4NL_VALUES[(packed >> (half * 4)) & 0xF];
}

static inline float iq4_xs_get(const uint8_t *w, int64_t index) {
    const uint8_t *blk = w + (index / QK_K) * IQ4_XS_BYTES;
    int within_block = (int)(index % QK_K);
    int g = within_block / 32;
    float d = jo_f16_to_f32(read_u16(blk));
    return iq4_xs_decode(blk, iq4_xs_group_scale(blk, d, g), g, within_block % 32);
}

float jo_get_float(int type, const uint8_t *w, int64_t index) {
    switch (type) {
        case JO_Q4_1: return q4_1_get(w, index);
        case JO_Q5_0: return q5_0_get(w, index);
        case JO_IQ4_XS: return iq4_xs_get(w, index);
        case JO_Q8_0: return q8_0_get(w, index);
        case JO_Q4_0: return q4_0_get(w, index);
        case JO_Q4_K: return q4_k_get(w, index);
        case JO_Q6_K: return q6_k_get(w, index);
        case JO_Q5_K: return q5_k_get(w, index);
        default: return NAN;
    }
}

void jo_dequant(int type, const uint8_t *w, int64_t n, float *out) {
    for (int64_t i = 0; i < n; i++) out[i] = jo_get_float(type, w, i);
}

/*
 * The reference states each decode a second time, in its device kernels, and its unit tests hold
 * the two wordings bit-equal.  Restated from those so the first wording can be checked against
 * something that was not typed from the same lines:
 *   Q4_0  J/backend/tornado/kernels/TransformerComputeKernelsQ4_0.java:72-79
 *   Q4_K  J/backend/tornado/kernels/TransformerComputeKernelsQ4_K.java:77-104
 *   Q8_0  src/test/java/.../kernels/QuantizedDeviceDecodeParityTest.java:349-358
 */
float jo_get_float_alt(int type, const uint8_t *w, int64_t index) {
    if (type == JO_Q8_0) {
        const uint8_t *blk = w + (index / 32) * Q8_0_BYTES;
        return jo_f16_to_f32(read_u16(blk)) * (float)(int8_t)blk[2 + index % 32];
    }
    if (type == JO_Q4_0) {
        const uint8_t *blk = w + (index / 32) * Q4_0_BYTES;
        int within = (int)(index % 32);
        float d = jo_f16_to_f32(read_u16(blk));
        int half = within / 16;
        int packed = blk[2 + within - half * 16];
        int q = (half == 0) ? (packed & 0xF) : ((packed >> 4) & 0xF);
        return d * (float)(q - 8);
    }
    if (type == JO_Q4_K) {
        const uint8_t *blk = w + (index / 256) * Q4_K_BYTES;
        int within = (int)(index % 256);
        float d = jo_f16_to_f32(read_u16(blk));
        float dmin = jo_f16_to_f32(read_u16(blk + 2));
        int pair = within / 64;
        int pos = within - pair * 64;
        int high = pos / 32;
        int sub = pair * 2 + high;
        int qb = blk[16 + pair * 32 + (pos - high * 32)];
        int q = (high == 0) ? (qb & 0xF) : ((qb >> 4) & 0xF);
        const uint8_t *s = blk + 4;
        int sc, m;
        if (sub < 4) {
            sc = s[sub] & 63;
            m = s[sub + 4] & 63;
        } else {
            int low = s[sub + 4];
            int hi = s[sub - 4];
            sc = (low & 0xF) | ((hi >> 6) << 4);
            m = ((low >> 4) & 0xF) | ((s[sub] >> 6) << 4);
        }
        float a = d * (float)sc;
        a = a * (float)q;
        float b = dmin * (float)m;
        return a - b;
    }
    if (type == JO_Q5_K) {
        /* J/backend/tornado/kernels/TransformerComputeKernelsQ5_K.java:144-220 */
        const uint8_t *blk = w + (index / 256) * Q5_K_BYTES;
        int within = (int)(index % 256);
        float d = jo_f16_to_f32(read_u16(blk));
        float dmin = jo_f16_to_f32(read_u16(blk + 2));
        int pair = within / 64;
        int pos_in_pair = within - pair * 64;
        int high_nibble = pos_in_pair / 32;
        int sub = pair * 2 + high_nibble;
        int pos = pos_in_pair - high_nibble * 32;
        int qs = blk[48 + pair * 32 + pos] & 0xFF;
        int q = high_nibble == 0 ? (qs & 0xF) : ((qs >> 4) & 0xF);
        int bits = blk[16 + pos] & 0xFF;
        if (pair >= 2) bits >>= 4;
        if ((pair & 1) == 1) bits >>= 2;
        if (high_nibble == 1) bits >>= 1;
        q += (bits & 1) * 16;
        const uint8_t *s = blk + 4;
        int sc, m;
        if (sub < 4) {
            sc = s[sub] & 63;
            m = s[sub + 4] & 63;
        } else {
            sc = (s[sub + 4] & 0xF) | ((s[sub - 4] >> 6) << 4);
            m = ((s[sub + 4] >> 4) & 0xF) | ((s[sub] >> 6) << 4);
        }
        float a = d * (float)sc;
        a = a * (float)q;
        float b = dmin * (float)m;
        return a - b;
    }
    if (type == JO_Q4_1) {
        /* J/backend/tornado/kernels/TransformerComputeKernelsQ4_1.java:59-67 */
        const uint8_t *blk = w + (index / 32) * Q4_1_BYTES;
        int within = (int)(index % 32);
        float d = jo_f16_to_f32(read_u16(blk));
        float m = jo_f16_to_f32(read_u16(blk + 2));
        int half = within / 16;
        int packed = blk[4 + (within - half * 16)] & 0xFF;
        int q = (half == 0) ? (packed & 0xF) : ((packed >> 4) & 0xF);
        float a = d * (float)q;
        return a + m;
    }
    if (type == JO_Q5_0) {
        /* J/backend/tornado/kernels/TransformerComputeKernelsQ5_0.java:56-70: the fifth bits are
           read as two 16-bit halves */
        const uint8_t *blk = w + (index / 32) * Q5_0_BYTES;
        int within = (int)(index % 32);
        float d = jo_f16_to_f32(read_u16(blk));
        uint32_t qh = (uint32_t)read_u16(blk + 2) | ((uint32_t)read_u16(blk + 4) << 16);
        int half = within / 16;
        int packed = blk[6 + within - half * 16] & 0xFF;
        int q = ((packed >> (half * 4)) & 0xF) | (int)(((qh >> within) & 1u) << 4);
        return d * (float)(q - 16);
    }
    if (type == JO_IQ4_XS) {
        /* J/backend/tornado/kernels/TransformerComputeKernelsIQ4_XS.java:62-96: the table as four
           little-endian words of four signed bytes */
        const uint8_t *blk = w + (index / 256) * IQ4_XS_BYTES;
        int within_block = (int)(index % 256);
        int g = within_block >> 5;
        int within = within_block & 31;
        int half = within >> 4;
        int packed = blk[8 + (g << 4) + (within & 15)] & 0xFF;
        int scales_h = read_u16(blk + 2);
        int low = blk[4 + (g >> 1)] & 0xFF;
        int ls = ((low >> ((g & 1) << 2)) & 0xF) | (((scales_h >> (g << 1)) & 3) << 4);
        float dl = jo_f16_to_f32(read_u16(blk)) * (float)(ls - 32);
        int q = (packed >> (half << 2)) & 0xF;
        uint32_t word = q < 8 ? (q < 4 ? 0xBFAD9881u : 0xF6EADDCFu) : (q < 12 ? 0x26190D01u : 0x71594535u);
        int kvalue = (int)(int8_t)(word >> ((q & 3) << 3));
        return dl * (float)kvalue;
    }
    if (type == JO_Q6_K) {
        /* J/backend/tornado/kernels/TransformerComputeKernelsQ6_K.java:195-232 */
        const uint8_t *blk = w + (index / 256) * Q6_K_BYTES;
        int within = (int)(index % 256);
        float d = jo_f16_to_f32(read_u16(blk + 208));
        int half_index = within / 128;
        int pos_in_half = within - half_index * 128;
        int group = pos_in_half / 32;
        int pos = pos_in_half - group * 32;
        int ql_base = half_index * 64, qh_base = 128 + half_index * 32, sc_base = 192 + half_index * 8;
        int is = pos / 16;
        int qh = blk[qh_base + pos] & 0xFF;
        int second_plane = group & 1, high_nibble = group >> 1;
        int ql = blk[ql_base + second_plane * 32 + pos] & 0xFF;
        int low_bits = high_nibble ? ((ql >> 4) & 0xF) : (ql & 0xF);
        int high_pair = (qh >> (2 * group)) & 3;
        int q = (low_bits | (high_pair << 4)) - 32;
        int scale = blk[sc_base + is + group * 2] & 0xFF;
        if (scale > 127) scale -= 256;
        float a = d * (float)scale;
        return a * (float)q;
    }
    return NAN;
}

/* ---- dot products -------------------------------------------------------------------------- */

/* J/tensor/standard/FloatTensor.java:110-117 */
static float scalar_dot(int type, const uint8_t *w, int64_t this_offset, const float *x,
                        int64_t that_offset, int64_t size) {
    float result = 0.0f;
    switch (type) {
        case JO_Q8_0:
            for (int64_t j = 0; j < size; j++) {
                float p = q8_0_get(w, this_offset + j) * x[that_offset + j];
                result += p;
            }
            break;
        case JO_Q4_0:
            for (int64_t j = 0; j < size; j++) {
                float p = q4_0_get(w, this_offset + j) * x[that_offset + j];
                result += p;
            }
            break;
        case JO_Q4_K:
            for (int64_t j = 0; j < size; j++) {
                float p = q4_k_get(w, this_offset + j) * x[that_offset + j];
                result += p;
            }
            break;
        case JO_Q5_K:   /* Q5_KFloatTensor.dot is scalarDot */
            for (int64_t j = 0; j < size; j++) {
                float p = q5_k_get(w, this_offset + j) * x[that_offset + j];
                result += p;
            }
            break;
        case JO_Q4_1:
            for (int64_t j = 0; j < size; j++) {
                float p = q4_1_get(w, this_offset + j) * x[that_offset + j];
                result += p;
            }
            break;
        case JO_Q5_0:
            for (int64_t j = 0; j < size; j++) {
                float p = q5_0_get(w, this_offset + j) * x[that_offset + j];
                result += p;
            }
            break;
        case JO_IQ4_XS:
            for (int64_t j = 0; j < size; j++) {
                float p = iq4_xs_get(w, this_offset + j) * x[that_offset + j];
                result += p;
            }
            break;
        case JO_Q6_K:   /* Q6_KFloatTensor.dot :124-127 is scalarDot */
            for (int64_t j = 0; j < size; j++) {
                float p = q6_k_get(w, this_offset + j) * x[that_offset + j];
                result += p;
            }
            break;
        default:
            return NAN;
    }
    return result;
}

/*
 * FloatVector.reduceLanes(ADD).  The JDK leaves the association open; its portable fallback folds
 * the lanes in index order starting from zero, which is what is used here.
 */
static inline float reduce_lanes(const float *val, int lanes) {
    float r = 0.0f;
    for (int l = 0; l < lanes; l++) r += val[l];
    return r;
}

/*
 * One block step of the vector kernels, shared by Q8_0 and Q4_0 once the 32 weights of the block
 * are widened to float in element order wf[0..31]:
 *   256-bit  val = fma(((s0 + s1) + s2) + s3, d, val), s_k = x[8k..8k+7] * wf[8k..8k+7]
 *   128-bit  two such steps over elements 0..15 and 16..31 with four 4-lane slices each
 * J/tensor/standard/Q8_0FloatTensor.java:161-216, Q4_0FloatTensor.java:120-163.
 * For Q4_0 the element order is lo nibbles of bytes 0..15 then hi nibbles of bytes 0..15, which is
 * exactly (lo part 0, lo part 1, hi part 0, hi part 1) at 256 bits and (lo parts 0..3), (hi parts
 * 0..3) at 128 bits.
 */
static inline __attribute__((always_inline)) void
block_step_256(const float *wf, const float *x, float d, float *val) {
    for (int l = 0; l < 8; l++) {
        float s0 = x[l] * wf[l];
        float s1 = x[8 + l] * wf[8 + l];
        float s2 = x[16 + l] * wf[16 + l];
        float s3 = x[24 + l] * wf[24 + l];
        float s = ((s0 + s1) + s2) + s3;
        val[l] = fmaf(s, d, val[l]);
    }
}

static inline __attribute__((always_inline)) void
block_step_128(const float *wf, const float *x, float d, float *val) {
    for (int i = 0; i < 2; i++) {
        const float *wh = wf + 16 * i;
        const float *xh = x + 16 * i;
        for (int l = 0; l < 4; l++) {
            float s0 = xh[l] * wh[l];
            float s1 = xh[4 + l] * wh[4 + l];
            float s2 = xh[8 + l] * wh[8 + l];
            float s3 = xh[12 + l] * wh[12 + l];
            float s = ((s0 + s1) + s2) + s3;
            val[l] = fmaf(s, d, val[l]);
        }
    }
}

/*
 * Q4_1's block step (J/tensor/standard/Q4_1FloatTensor.java:141-182): the same four products, summed
 * left to right, scaled into val by d; then the four activation slices, summed left to right,
 * scaled into val by the block's minimum.
 */
static inline __attribute__((always_inline)) void
block_step_256_affine(const float *wf, const float *x, float d, float m, float *val) {
    for (int l = 0; l < 8; l++) {
        float products = ((x[l] * wf[l] + x[8 + l] * wf[8 + l]) + x[16 + l] * wf[16 + l]) + x[24 + l] * wf[24 + l];
        float activations = ((x[l] + x[8 + l]) + x[16 + l]) + x[24 + l];
        val[l] = fmaf(products, d, val[l]);
        val[l] = fmaf(activations, m, val[l]);
    }
}

static inline __attribute__((always_inline)) void
block_step_128_affine(const float *wf, const float *x, float d, float m, float *val) {
    for (int i = 0; i < 2; i++) {
        const float *wh = wf + 16 * i;
        const float *xh = x + 16 * i;
        for (int l = 0; l < 4; l++) {
            float products = ((xh[l] * wh[l] + xh[4 + l] * wh[4 + l]) + xh[8 + l] * wh[8 + l]) + xh[12 + l] * wh[12 + l];
            float activations = ((xh[l] + xh[4 + l]) + xh[8 + l]) + xh[12 + l];
            val[l] = fmaf(products, d, val[l]);
            val[l] = fmaf(activations, m, val[l]);
        }
    }
}

static inline __attribute__((always_inline)) void widen_q4_1(const uint8_t *blk, float *wf) {
    for (int i = 0; i < 16; i++) {
        wf[i] = (float)(blk[4 + i] & 0xF);       /* unsigned nibbles: no recentring */
        wf[16 + i] = (float)(blk[4 + i] >> 4);
    }
}

static inline __attribute__((always_inline)) void widen_q8_0(const uint8_t *blk, float *wf) {
    for (int i = 0; i < 32; i++) wf[i] = (float)(int8_t)blk[2 + i];
}

static inline __attribute__((always_inline)) void widen_q4_0(const uint8_t *blk, float *wf) {
    for (int i = 0; i < 16; i++) {
        /* byte lanes: (b & 0xF) - 8 and (b >>> 4) - 8, then castShape widens the signed byte */
        int8_t lo = (int8_t)((blk[2 + i] & 0xF) - 8);
        int8_t hi = (int8_t)((blk[2 + i] >> 4) - 8);
        wf[i] = (float)lo;
        wf[16 + i] = (float)hi;
    }
}

/* J/tensor/standard/Q8_0FloatTensor.java:142-229, Q4_0FloatTensor.java:90-174, Q4_1FloatTensor.java:105-192 */
static inline __attribute__((always_inline)) float
vector_dot_body(int type, int bits, const uint8_t *w, int64_t this_offset, const float *x,
           int64_t that_offset, int64_t size) {
    const int block_bytes = (type == JO_Q8_0) ? Q8_0_BYTES : (type == JO_Q4_1) ? Q4_1_BYTES : Q4_0_BYTES;
    float result = 0.0f;
    int64_t j = 0;
    int64_t alignment_bound = (-this_offset) & (Q_BLOCK - 1);
    if (alignment_bound > size) alignment_bound = size;
    if (alignment_bound > 0) {
        result += scalar_dot(type, w, this_offset, x, that_offset, alignment_bound);
        j += alignment_bound;
    }
    float val[8] = {0, 0, 0, 0, 0, 0, 0, 0};
    int64_t block_offset = (this_offset + j) / Q_BLOCK * block_bytes;
    int64_t upper_bound = size / Q_BLOCK * Q_BLOCK;
    float wf[32];
    /* the reference loop tests j < upperBound only; j + 32 <= size is added so that a misaligned
       offset (which no matmul caller produces) cannot read past the slice */
    for (; j < upper_bound && j + Q_BLOCK <= size; j += Q_BLOCK, block_offset += block_bytes) {
        const uint8_t *blk = w + block_offset;
        float d = jo_f16_to_f32(read_u16(blk));
        if (type == JO_Q4_1) {
            float m = jo_f16_to_f32(read_u16(blk + 2));
            widen_q4_1(blk, wf);
            if (bits == 256) block_step_256_affine(wf, x + that_offset + j, d, m, val);
            else block_step_128_affine(wf, x + that_offset + j, d, m, val);
            continue;
        }
        if (type == JO_Q8_0) widen_q8_0(blk, wf); else widen_q4_0(blk, wf);
        if (bits == 256) block_step_256(wf, x + that_offset + j, d, val);
        else block_step_128(wf, x + that_offset + j, d, val);
    }
    result += reduce_lanes(val, bits == 256 ? 8 : 4);
    if (j < size) {
        result += scalar_dot(type, w, this_offset + j, x, that_offset + j, size - j);
    }
    return result;
}

/* The same body compiled twice: once for AVX2+FMA hosts, once for anything else. */
__attribute__((target("avx2,fma"))) static float
vector_dot_avx2(int type, int bits, const uint8_t *w, int64_t this_offset, const float *x,
                int64_t that_offset, int64_t size) {
    return vector_dot_body(type, bits, w, this_offset, x, that_offset, size);
}

static float vector_dot_generic(int type, int bits, const uint8_t *w, int64_t this_offset,
                                const float *x, int64_t that_offset, int64_t size) {
    return vector_dot_body(type, bits, w, this_offset, x, that_offset, size);
}

static float vector_dot(int type, int bits, const uint8_t *w, int64_t this_offset, const float *x,
                        int64_t that_offset, int64_t size) {
    static int have_avx2 = -1;
    if (have_avx2 < 0) have_avx2 = __builtin_cpu_supports("avx2") && __builtin_cpu_supports("fma");
    return have_avx2 ? vector_dot_avx2(type, bits, w, this_offset, x, that_offset, size)
                     : vector_dot_generic(type, bits, w, this_offset, x, that_offset, size);
}

/*
 * Q5_0FloatTensor.dot (J/tensor/standard/Q5_0FloatTensor.java:87-112) and IQ4_XSFloatTensor.dot
 * (IQ4_XSFloatTensor.java:102-126): no vector kernel, but not scalarDot either -- a block's (Q5_0)
 * or a group's (IQ4_XS) 32 products are summed on their own from zero and that sum is added to the
 * result; elements before the first whole block and after the last one go through scalarDot.
 */
static float block_sum_dot(int type, const uint8_t *w, int64_t this_offset, const float *x,
                           int64_t that_offset, int64_t size) {
    const int elems = (type == JO_Q5_0) ? Q_BLOCK : QK_K;
    const int bytes = (type == JO_Q5_0) ? Q5_0_BYTES : IQ4_XS_BYTES;
    float result = 0.0f;
    int64_t j = 0;
    int64_t alignment_bound = (-this_offset) & (elems - 1);
    if (alignment_bound > size) alignment_bound = size;
    if (alignment_bound > 0) {
        result += scalar_dot(type, w, this_offset, x, that_offset, alignment_bound);
        j += alignment_bound;
    }
    int64_t block_offset = (this_offset + j) / elems * bytes;
    for (; j + elems <= size; j += elems, block_offset += bytes) {
        const uint8_t *blk = w + block_offset;
        float d = jo_f16_to_f32(read_u16(blk));
        if (type == JO_Q5_0) {
            uint32_t qh = q5_0_high_bits(blk);
            float block = 0.0f;
            for (int i = 0; i < Q_BLOCK; i++) {
                float p = q5_0_decode(blk, d, qh, i) * x[that_offset + j + i];
                block += p;
            }
            result += block;
        } else {
            for (int g = 0; g < QK_K / 32; g++) {
                float dl = iq4_xs_group_scale(blk, d, g);
                float group = 0.0f;
                for (int i = 0; i < 32; i++) {
                    float p = iq4_xs_decode(blk, dl, g, i) * x[that_offset + j + g * 32 + i];
                    group += p;
                }
                result += group;
            }
        }
    }
    if (j < size) result += scalar_dot(type, w, this_offset + j, x, that_offset + j, size - j);
    return result;
}

/*
 * Q8_0FloatTensor.dotQ8Activation (J/tensor/standard/Q8_0FloatTensor.java:107-140), the branch
 * Q8_0FloatTensor.dot takes under -Djitllm.quantizeActivation=true (:86-93; off by default).  Per
 * block of 32: the activations' largest magnitude over 127 is the quantization scale; the int8
 * values are derived with that fp32 scale (x * (1 / scale), rounded half away from zero through
 * `(int)(s + copySign(0.5f, s))`), the scale that multiplies the integer sum is the same number
 * rounded to binary16 and back; `result += isum * (wScale * aScale)` block after block.  Offsets
 * and sizes are multiples of 32 for every caller; a remainder is dropped, as there.
 */
/* Java's (int) of a float: NaN gives 0 and the range saturates; C leaves both undefined. */
static int32_t java_float_to_int(float v) {
    if (v != v) return 0;
    if (v >= 2147483648.0f) return INT32_MAX;
    if (v <= -2147483648.0f) return INT32_MIN;
    return (int32_t)v;
}

static float q8_activation_dot(const uint8_t *w, int64_t this_offset, const float *x, int64_t that_offset,
                               int64_t size) {
    float result = 0.0f;
    const int64_t nblocks = size / 32;
    for (int64_t b = 0; b < nblocks; b++) {
        const int64_t elem_base = b * 32;
        const uint8_t *blk = w + (this_offset + elem_base) / 32 * 34;
        const float w_scale = jo_f16_to_f32((uint16_t)(blk[0] | (blk[1] << 8)));
        float amax = 0.0f;
        for (int i = 0; i < 32; i++) {
            const float av = fabsf(x[that_offset + elem_base + i]);
            if (av > amax) amax = av;
        }
        const float quantization_scale = amax / 127.0f;
        const float a_scale = jo_f16_to_f32(jo_f32_to_f16(quantization_scale));
        const float a_inv = quantization_scale != 0.0f ? 1.0f / quantization_scale : 0.0f;
        int32_t isum = 0;
        for (int i = 0; i < 32; i++) {
            const float s = x[that_offset + elem_base + i] * a_inv;
            const float shifted = s + copysignf(0.5f, s);
            const int32_t aq = java_float_to_int(shifted);
            isum += aq * (int32_t)(int8_t)blk[2 + i];
        }
        const float scales = w_scale * a_scale;
        result += (float)isum * scales;
    }
    return result;
}

/*
 * Q8_0FloatTensor.dot (J/tensor/standard/Q8_0FloatTensor.java:89-99), Q4_0FloatTensor.dot
 * (Q4_0FloatTensor.java:82-88), Q4_KFloatTensor.dot (Q4_KFloatTensor.java:124-127).  The flavour
 * is the branch a JVM would take: vector kernels exist for 128- and 256-bit species only
 * (FloatTensor.java:33-36); Q4_K is always scalar.
 */
float jo_dot(int type, int flavour, const uint8_t *w, int64_t this_offset, const float *x,
             int64_t that_offset, int64_t size) {
    /* Q5_0 and IQ4_XS have one dot for every JVM (the flavour only matters to the vector kernels) */
    if (type == JO_Q5_0 || type == JO_IQ4_XS) return block_sum_dot(type, w, this_offset, x, that_offset, size);
    /* the quantized-activation branch exists in Q8_0FloatTensor only and comes before the others */
    if (type == JO_Q8_0 && flavour == JO_DOT_Q8ACT) return q8_activation_dot(w, this_offset, x, that_offset, size);
    if ((type == JO_Q8_0 || type == JO_Q4_0 || type == JO_Q4_1) && (flavour == JO_DOT_VEC128 || flavour == JO_DOT_VEC256)) {
        return vector_dot(type, flavour, w, this_offset, x, that_offset, size);
    }
    return scalar_dot(type, w, this_offset, x, that_offset, size);
}

/* J/tensor/standard/FloatTensor.java:123-125 + J/auxiliary/Parallel.java:9-11 */
void jo_matmul(int type, int flavour, const uint8_t *w, const float *x, float *out, int dim0,
               int dim1, int nthreads) {
    if (nthreads < 1) nthreads = 1;
#pragma omp parallel for schedule(static) num_threads(nthreads)
    for (int i = 0; i < dim0; i++) {
        out[i] = jo_dot(type, flavour, w, (int64_t)i * dim1, x, 0, dim1);
    }
}

/* J/tensor/standard/FloatTensor.java:127-140 + J/auxiliary/Parallel.java:13-20 */
void jo_matmul_batch(int type, int flavour, const uint8_t *w, const float *X, float *out,
                     int context, int dim0, int dim1, int nthreads) {
    if (nthreads < 1) nthreads = 1;
    int64_t total = (int64_t)dim0 * context;
#pragma omp parallel for schedule(static) num_threads(nthreads)
    for (int64_t ti = 0; ti < total; ti++) {
        int idx_arr = (int)(ti / dim0);
        int i = (int)(ti % dim0);
        out[(int64_t)idx_arr * dim0 + i] =
            jo_dot(type, flavour, w, (int64_t)i * dim1, X + (int64_t)idx_arr * dim1, 0, dim1);
    }
}

/* J/inference/op/CpuOperations.java:255-260 */
void jo_swiglu(float *gate, const float *up, int64_t n) {
    for (int64_t i = 0; i < n; i++) {
        float value = gate[i];
        float act = value / (float)(1.0 + exp(-(double)value));
        gate[i] = act * up[i];
    }
}

/* ---- the steps on either side of a projection ---------------------------------------------- */

/*
 * J/inference/op/CpuOperations.java:60-66 with FloatTensor.reduce (J/tensor/standard/FloatTensor.java:
 * 147-153): ss = sum x_i^2 sequentially in fp32 from 0f; ss /= size; ss += eps;
 * ss = (float)(1.0 / Math.sqrt(ss)).
 */
float jo_rms_scale(const float *x, int64_t n, float eps) {
    float ss = 0.0f;
    for (int64_t i = 0; i < n; i++) {
        float sq = x[i] * x[i];   /* acc + xi * xi: product rounded, then the sum (no FMA in the lambda) */
        ss = ss + sq;
    }
    ss /= (float)n;
    ss += eps;
    return (float)(1.0 / sqrt((double)ss));
}

/* J/inference/op/CpuOperations.java:67-72: out[i] = weight[i] * (ss * x[i]) */
void jo_rmsnorm(float *out, const float *x, const float *weight, int64_t n, float eps) {
    float ss = jo_rms_scale(x, n, eps);
    for (int64_t i = 0; i < n; i++) {
        float scaled = ss * x[i];
        out[i] = weight[i] * scaled;
    }
}

/*
 * The batched prefill's normalisation, which hands the projections fp16 activations:
 * batchedRmsReduceParallel (J/backend/tornado/kernels/TransformerBatchPrefillKernels.java:1480-1510)
 * with its local size of 256 -- work item t adds the squares of elements t, t + 256, ... in turn,
 * the 256 partial sums fold as the binary tree partial[t] += partial[t + s], s = 128 ... 1, and
 * scale = 1.0f / sqrt(partial[0] / dim + eps) in fp32 -- then batchedRmsApplyFP16 (:59-72):
 * out = FP16(rmsWeights[i] * scale * x[i]), the products taken left to right and rounded to fp32,
 * the result to the nearest fp16.  `scales` (one per row) may be null.  With `delta` the pending
 * residual add comes first, as in batchedRmsReduceFusedResidual (:1519-1551): x[b][i] += delta[b][i]
 * is written back and the sums run over the updated row.
 */
void jo_batched_rms_apply_f16(float *x, const float *delta, const float *weight, float eps, int64_t rows,
                              int64_t n, float *scales, uint16_t *out) {
    enum { LOCAL = 256 };
    for (int64_t b = 0; b < rows; b++) {
        float *row = x + b * n;
        if (delta)
            for (int64_t i = 0; i < n; i++) row[i] = row[i] + delta[b * n + i];
        float partial[LOCAL];
        for (int t = 0; t < LOCAL; t++) {
            float ss = 0.0f;
            for (int64_t i = t; i < n; i += LOCAL) {
                float sq = row[i] * row[i];
                ss = ss + sq;
            }
            partial[t] = ss;
        }
        for (int s = LOCAL / 2; s > 0; s >>= 1)
            for (int t = 0; t < s; t++) partial[t] = partial[t] + partial[t + s];
        float m = partial[0] / (float)n;
        m = m + eps;
        float scale = 1.0f / sqrtf(m);
        if (scales) scales[b] = scale;
        for (int64_t i = 0; i < n; i++) {
            float ws = weight[i] * scale;
            float r = ws * row[i];
            out[b * n + i] = jo_f32_to_f16(r);
        }
    }
}

/* J/tensor/standard/FloatTensor.java:168-181: the first maximum; a NaN never wins a comparison */
int64_t jo_argmax(const float *x, int64_t n) {
    int64_t max_index = 0;
    float max_value = x[0];
    for (int64_t i = 0; i < n; i++) {
        float f = x[i];
        if (f > max_value) {
            max_value = f;
            max_index = i;
        }
    }
    return max_index;
}

/* ---- int8 activation path (the arithmetic the reference's int8 GEMM defines) -------------- */

/*
 * J/backend/tornado/kernels/Int8GemmKernels.java:96-129 (quantizeActivationsQ8Warp):
 * d = amax / 127; q = 0 if d == 0, else round-half-away(x * (127 / amax)) clamped to +-127, with
 * the (x / amax) * 127 form below RECIPROCAL_FINITE_AMAX = 4e-37.
 */
void jo_quantize_q8(const float *x, int8_t *q, float *scales, int64_t rows, int64_t k) {
    int64_t blocks = rows * k / 32;
    for (int64_t b = 0; b < blocks; b++) {
        const float *xb = x + b * 32;
        float amax = 0.0f;
        for (int i = 0; i < 32; i++) {
            float a = fabsf(xb[i]);
            if (a > amax) amax = a;
        }
        float d = amax / 127.0f;
        for (int i = 0; i < 32; i++) {
            int qv = 0;
            if (d > 0.0f) {
                float v;
                if (amax >= 4.0e-37f) v = xb[i] * (127.0f / amax);
                else v = (xb[i] / amax) * 127.0f;
                qv = (int)floorf(fabsf(v) + 0.5f);
                if (qv > 127) qv = 127;
                if (v < 0.0f) qv = -qv;
            }
            q[b * 32 + i] = (int8_t)qv;
        }
        scales[b] = d;
    }
}

/*
 * J/backend/tornado/kernels/Int8GemmKernels.java:17-23: each 32-block's dot product exact in
 * int32; acc = fma((float)dot * dA, dW, acc) over the blocks in k order.  Weights are Q8_0 quants
 * or Q4_0 nibbles recentred to q - 8; dW is the fp16 block scale widened to fp32.
 */
void jo_gemm_int8_block_scaled(int type, const int8_t *aq, const float *ascale, const uint8_t *w,
                               float *out, int m, int n, int k, int nthreads) {
    if (nthreads < 1) nthreads = 1;
    const int kb = k / 32;
    const int block_bytes = jo_block_bytes(type);
#pragma omp parallel for schedule(static) num_threads(nthreads)
    for (int col = 0; col < n; col++) {
        for (int row = 0; row < m; row++) {
            float acc = 0.0f;
            for (int b = 0; b < kb; b++) {
                const uint8_t *blk = w + ((int64_t)col * kb + b) * block_bytes;
                float dw = jo_f16_to_f32(read_u16(blk));
                const int8_t *a = aq + (int64_t)row * k + b * 32;
                int32_t dot = 0;
                if (type == JO_Q8_0) {
                    for (int i = 0; i < 32; i++) dot += (int32_t)a[i] * (int8_t)blk[2 + i];
                } else {
                    for (int i = 0; i < 16; i++) {
                        dot += (int32_t)a[i] * ((blk[2 + i] & 0xF) - 8);
                        dot += (int32_t)a[16 + i] * ((blk[2 + i] >> 4) - 8);
                    }
                }
                float t = (float)dot * ascale[(int64_t)row * kb + b];
                acc = fmaf(t, dw, acc);
            }
            out[(int64_t)row * n + col] = acc;
        }
    }
}

/* ---- the packed-integer decode path ("dp4a") --------------------------------------------------- */

/*
 * quantizeActivationQ8Blocks, J/backend/tornado/kernels/TransformerComputeKernelsQ4_0.java:287-341:
 * per block of 32, inverse = maxAbs > 0 ? 127 / maxAbs : 0; q = (int)(x * inverse + (+-0.5)) clamped
 * to [-127, 127]; scales[b] = maxAbs / 127; sums[b] = sum of the block's q.  (A Java (int) cast
 * sends NaN to 0 and saturates; both are spelled out, C leaves them undefined.)
 */
void jo_quantize_q8_blocks(const float *x, int64_t n, int8_t *q, float *scales, int32_t *sums) {
    for (int64_t b = 0; b < n / 32; b++) {
        const float *xb = x + b * 32;
        float max_abs = 0.0f;
        for (int i = 0; i < 32; i++) {
            float a = fabsf(xb[i]);
            if (a > max_abs) max_abs = a;   /* Math.max over a tree: order cannot matter */
        }
        float inverse = max_abs > 0.0f ? 127.0f / max_abs : 0.0f;
        int32_t sum = 0;
        for (int i = 0; i < 32; i++) {
            float scaled = xb[i] * inverse;
            float t = scaled + (scaled >= 0.0f ? 0.5f : -0.5f);
            int qi;
            if (t != t) qi = 0;
            else if (t >= 128.0f) qi = 127;
            else if (t <= -128.0f) qi = -127;
            else qi = (int)t;
            if (qi > 127) qi = 127;
            if (qi < -127) qi = -127;
            q[b * 32 + i] = (int8_t)qi;
            sum += qi;
        }
        scales[b] = max_abs / 127.0f;
        sums[b] = sum;
    }
}

/*
 * One row of the packed projections, the blocks (Q4_K: units of 16 weights) taken in order:
 *   Q8_0  partial += weightScale * xScale * dot               TransformerComputeKernelsQ8_0DP4A.java:35-68
 *   Q4_0  partial += weightScale * xScale * (dot - 8 * xSum)  TransformerComputeKernelsQ4_0.java:487-506
 *   Q4_K  partial += dAll * (scale0 * xs0 * dot0 + scale1 * xs1 * dot1)
 *                    - first * dMin * (min0 * xs0 * sum0 + min1 * xs1 * sum1)
 *                                                             TransformerComputeKernelsQ4_K.java:599-668
 * with every dot an exact int32 sum and Java's left-to-right float products.  The reference's
 * kernels deal the blocks to lanes and fold the lanes' partials with shuffles, an order that
 * depends on the launch's lane count; the sequential order here is one of them, and comparisons
 * are held to a rounding tolerance, not to bit equality.
 */
static float packed_row(int type, const uint8_t *row, const int8_t *q, const float *xs, const int32_t *xsum, int n) {
    float partial = 0.0f;
    if (type == JO_Q8_0 || type == JO_Q4_0) {
        const int bytes = type == JO_Q8_0 ? Q8_0_BYTES : Q4_0_BYTES;
        for (int b = 0; b < n / 32; b++) {
            const uint8_t *blk = row + (int64_t)b * bytes;
            float weight_scale = jo_f16_to_f32(read_u16(blk));
            const int8_t *a = q + b * 32;
            int32_t dot = 0;
            if (type == JO_Q8_0) {
                for (int i = 0; i < 32; i++) dot += (int32_t)(int8_t)blk[2 + i] * a[i];
                float t = weight_scale * xs[b];
                partial += t * (float)dot;
            } else {
                for (int i = 0; i < 16; i++) {
                    dot += (int32_t)(blk[2 + i] & 0xF) * a[i];
                    dot += (int32_t)(blk[2 + i] >> 4) * a[16 + i];
                }
                float t = weight_scale * xs[b];
                partial += t * (float)(dot - 8 * xsum[b]);
            }
        }
        return partial;
    }
    for (int unit = 0; unit < n / 16; unit++) {
        int super_block = unit >> 4, in_block = unit & 15, pair = in_block >> 2, quarter = in_block & 3;
        const uint8_t *blk = row + (int64_t)super_block * Q4_K_BYTES;
        float d_all = jo_f16_to_f32(read_u16(blk));
        float d_min = jo_f16_to_f32(read_u16(blk + 2));
        int scale0 = q4_k_scale(2 * pair, blk + 4), min0 = q4_k_min(2 * pair, blk + 4);
        int scale1 = q4_k_scale(2 * pair + 1, blk + 4), min1 = q4_k_min(2 * pair + 1, blk + 4);
        const uint8_t *qs = blk + 16 + pair * 32 + quarter * 8;
        int block0 = super_block * 8 + pair * 2, block1 = block0 + 1;
        const int8_t *a0 = q + block0 * 32 + quarter * 8, *a1 = q + block1 * 32 + quarter * 8;
        int32_t dot0 = 0, dot1 = 0;
        for (int i = 0; i < 8; i++) {
            dot0 += (int32_t)(qs[i] & 0xF) * a0[i];
            dot1 += (int32_t)(qs[i] >> 4) * a1[i];
        }
        float xs0 = xs[block0], xs1 = xs[block1];
        float first = (float)(1 - (quarter < 1 ? quarter : 1));
        float t0 = (float)scale0 * xs0;
        t0 = t0 * (float)dot0;
        float t1 = (float)scale1 * xs1;
        t1 = t1 * (float)dot1;
        float lhs = d_all * (t0 + t1);
        float m0 = (float)min0 * xs0;
        m0 = m0 * (float)xsum[block0];
        float m1 = (float)min1 * xs1;
        m1 = m1 * (float)xsum[block1];
        float rhs = first * d_min;
        rhs = rhs * (m0 + m1);
        partial += lhs - rhs;
    }
    return partial;
}

void jo_matmul_q8x(int type, const uint8_t *w, const int8_t *q, const float *scales, const int32_t *sums,
                   float *out, int dim0, int dim1, int nthreads) {
    if (nthreads < 1) nthreads = 1;
    const int64_t row_bytes = (int64_t)dim1 / jo_block_elems(type) * jo_block_bytes(type);
#pragma omp parallel for schedule(static) num_threads(nthreads)
    for (int i = 0; i < dim0; i++) out[i] = packed_row(type, w + i * row_bytes, q, scales, sums, dim1);
}

/* ---- java.util.Random (the generator the reference's test fixtures are drawn from) --------- */

#define JR_MULT 0x5DEECE66DLL
#define JR_MASK ((1LL << 48) - 1)

void jo_jrandom_init(jo_jrandom *r, int64_t seed) {
    r->seed = (seed ^ JR_MULT) & JR_MASK;
    r->have_next_next_gaussian = 0;
    r->next_next_gaussian = 0.0;
}

static inline int32_t jr_next(jo_jrandom *r, int bits) {
    r->seed = (int64_t)(((uint64_t)r->seed * (uint64_t)JR_MULT + 0xBULL) & (uint64_t)JR_MASK);
    return (int32_t)(r->seed >> (48 - bits));
}

int32_t jo_jrandom_next_int(jo_jrandom *r) { return jr_next(r, 32); }

int32_t jo_jrandom_next_int_bound(jo_jrandom *r, int32_t bound) {
    if (bound <= 0) return 0;
    int32_t v = jr_next(r, 31);
    int32_t m = bound - 1;
    if ((bound & m) == 0) return (int32_t)(((int64_t)bound * (int64_t)v) >> 31);
    int32_t u = v;
    /* reject while u - (u % bound) + m overflows int32 */
    while (1) {
        v = u % bound;
        int64_t t = (int64_t)u - v + m;
        if (t <= INT32_MAX) break;
        u = jr_next(r, 31);
    }
    return v;
}

int jo_jrandom_next_boolean(jo_jrandom *r) { return jr_next(r, 1) != 0; }

static inline double jr_next_double(jo_jrandom *r) {
    int64_t hi = (int64_t)jr_next(r, 26) << 27;
    int64_t lo = jr_next(r, 27);
    return (double)(hi + lo) * 0x1.0p-53;
}

double jo_jrandom_next_gaussian(jo_jrandom *r) {
    if (r->have_next_next_gaussian) {
        r->have_next_next_gaussian = 0;
        return r->next_next_gaussian;
    }
    double v1, v2, s;
    do {
        v1 = 2 * jr_next_double(r) - 1;
        v2 = 2 * jr_next_double(r) - 1;
        s = v1 * v1 + v2 * v2;
    } while (s >= 1 || s == 0);
    double multiplier = sqrt(-2 * log(s) / s);
    r->next_next_gaussian = v2 * multiplier;
    r->have_next_next_gaussian = 1;
    return v1 * multiplier;
}

void jo_jrandom_next_bytes(jo_jrandom *r, uint8_t *out, int64_t n) {
    int64_t i = 0;
    while (i < n) {
        int32_t rnd = jo_jrandom_next_int(r);
        int64_t take = n - i < 4 ? n - i : 4;
        while (take-- > 0) {
            out[i++] = (uint8_t)rnd;
            rnd >>= 8;
        }
    }
}

int32_t jo_java_string_hash(const char *s) {
    uint32_t h = 0;
    for (; *s; s++) h = 31u * h + (uint8_t)*s;
    return (int32_t)h;
}
