// Single-token projection over Q6_K, Q5_K, Q4_1, Q5_0 and IQ4_XS weights: out (+)= W . x.
//
// Files quantised "Q4_K_M" / "Q5_K_M" keep their vocabulary projection and some attention /
// feed-forward tensors in Q6_K, and the reference reads a projection "by its own representation,
// not the plan's" (J/backend/tornado/layers/type/q8_0/LogitsQ8_0Layer.java:92-96), so a K-quant
// model needs these kernels beside the Q4_K ones.  Replaces matrixVectorGenericQ6_K / Q5_K and
// their residual forms (J/backend/tornado/kernels/TransformerComputeKernelsQ6_K.java:548-590,
// TransformerComputeKernelsQ5_K.java); the arithmetic is the host tensors':
//   Q6_K  ql[128] | qh[64] | 16 signed scales | fp16 d          w = d * scale * (q - 32)
//         (J/tensor/standard/Q6_KFloatTensor.java:66-122)
//   Q5_K  fp16 d, dmin | 12 packed scale/min bytes | qh[32] | qs[128]   w = d * sc * q - dmin * m,
//         q = nibble + 16 * (bit 2 pair + nibble half of qh)  (Q5_KFloatTensor.java:78-122)
// and the types quantisers mix into Q4_0 / K-quant files (matrixVectorGenericQ4_1 / Q5_0 / IQ4_XS,
// TransformerComputeKernelsQ4_1.java:272-290, ...Q5_0.java:261-279, ...IQ4_XS.java:248-266):
//   Q4_1  fp16 d, m | 16 nibble bytes                w = d * q + m      (Q4_1FloatTensor.java:73-94)
//   Q5_0  fp16 d | 32 fifth bits | 16 nibble bytes   w = d * (q - 16)   (Q5_0FloatTensor.java:61-85)
//   IQ4_XS fp16 d | scales_h | scales_l[4] | qs[128] w = d * (ls - 32) * kvalues_iq4nl[q]
//         (IQ4_XSFloatTensor.java:72-100)
// whose 16 nibble bytes hold elements 0..15 of a group of 32 in their low halves and 16..31 in
// their high halves: a lane takes eight consecutive bytes of one group.
//
// One wave per weight row, sixteen lanes per super-block.  A lane reads eight consecutive bytes of
// the low-bit plane and the eight high-bit bytes of the same positions, which hold sixteen
// weights: eight consecutive ones in each of two groups of 32.  The values are put together a
// dword (four weights) at a time; the constant offset and the group's scale are applied to the
// group's partial sum, not to each weight.  The weights are read straight from global memory (a
// row's bytes are used once): the sixteen lanes of a super-block read its low-bit plane as one
// contiguous 128-byte run.  For the usual row lengths a lane's activations are the same in every
// row and stay in registers.
#include "jl_device.h"
#include "jl_internal.h"

namespace {

struct __attribute__((packed, aligned(2))) U32a2 { uint32_t v; };
struct __attribute__((packed, aligned(2))) U64a2 { uint32_t lo, hi; };

__device__ __forceinline__ float ub(uint32_t v, int k) { return (float)((v >> (8 * k)) & 0xFFu); }

// sum over the four bytes of q (values 0..255) times x
__device__ __forceinline__ float dot4(uint32_t q, const float4 x) {
    q = jl_opaque(q);   // keeps the four conversions byte selects of one register
    return fmaf(ub(q, 0), x.x, fmaf(ub(q, 1), x.y, fmaf(ub(q, 2), x.z, ub(q, 3) * x.w)));
}

template <int TYPE> struct Raw;

// Q6_K, lane j = (h, i) with h = j / 8: eight consecutive ql bytes -- lanes i < 4 of plane 0 (groups
// 0 and 2 of half h), lanes i >= 4 of plane 1 (groups 1 and 3) -- and the eight qh bytes of the
// same positions.
template <> struct Raw<JL_Q6_K> {
    U64a2 ql, qh;
    U64a2 s8;              // the half's 8 scales
    unsigned short d;
};
// Q5_K, lane j = (pair, i) with pair = j / 4: eight consecutive nibble bytes of the pair (sub-block
// 2 pair in the low nibbles, 2 pair + 1 in the high ones) and the eight fifth-bit bytes of the
// same positions; the header is d, dmin and the 12 scale / min bytes.
template <> struct Raw<JL_Q5_K> {
    uint2 qs, qh;
    uint4 hdr;
};
// Q4_1 / Q5_0 / IQ4_XS, lane j = (group, half) with group = j / 2: bytes 8 half .. 8 half + 7 of the
// group's sixteen.  Q4_1 blocks are 4-byte aligned, Q5_0 blocks 2-byte, IQ4_XS super-blocks 8-byte.
struct __attribute__((packed, aligned(4))) U64a4 { uint32_t lo, hi; };
template <> struct Raw<JL_Q4_1> {
    U64a4 qs;
    uint32_t dm;           // d, m
};
template <> struct Raw<JL_Q5_0> {
    U64a2 qs;
    U32a2 qh;
    unsigned short d;
};
template <> struct Raw<JL_IQ4_XS> {
    uint2 qs;
    uint2 hdr;             // d, scales_h | scales_l
};
// The sixteen activations that go with it: eight consecutive ones of the low-nibble group and
// eight of the high-nibble group, with -32 times their sums (the "- 32" of every weight, applied
// to the group's sum).
struct Xs {
    float4 x[4];
    float m32[2];   // the sum of each eight, times the constant the type takes off every weight:
                    // Q6_K -32, Q5_0 -16, IQ4_XS -128 (its table is used with 128 added); Q5_K and
                    // Q4_1, whose minimum is per block, the plain sums
};

template <int TYPE>
__device__ __forceinline__ Raw<TYPE> load_raw(const uint8_t *blk, int j) {
    Raw<TYPE> r;
    if constexpr (TYPE == JL_Q6_K) {
        const int h = j >> 3, i = j & 7;
        r.ql = *(const U64a2 *)(blk + 64 * h + 32 * (i >> 2) + 8 * (i & 3));
        r.qh = *(const U64a2 *)(blk + 128 + 32 * h + 8 * (i & 3));
        r.s8 = *(const U64a2 *)(blk + 192 + 8 * h);
        r.d = *(const unsigned short *)(blk + 208);
    } else if constexpr (TYPE == JL_Q5_K) {
        const int pair = j >> 2, i = j & 3;   // super-blocks are 176 bytes: everything is aligned
        r.hdr = *(const uint4 *)blk;
        r.qh = *(const uint2 *)(blk + 16 + 8 * i);
        r.qs = *(const uint2 *)(blk + 48 + 32 * pair + 8 * i);
    } else if constexpr (TYPE == JL_Q4_1) {
        const uint8_t *b = blk + 20 * (j >> 1);
        r.dm = *(const uint32_t *)b;
        r.qs = *(const U64a4 *)(b + 4 + 8 * (j & 1));
    } else if constexpr (TYPE == JL_Q5_0) {
        const uint8_t *b = blk + 22 * (j >> 1);
        r.d = *(const unsigned short *)b;
        r.qh = *(const U32a2 *)(b + 2);
        r.qs = *(const U64a2 *)(b + 6 + 8 * (j & 1));
    } else {
        r.hdr = *(const uint2 *)blk;
        r.qs = *(const uint2 *)(blk + 8 + 8 * j);
    }
    return r;
}

// first of the lane's sixteen activations inside its super-block; the second eight are 64 (Q6_K)
// or 32 (Q5_K) elements further on
template <int TYPE>
__device__ __forceinline__ Xs load_x(const float *x, int j) {
    Xs v;
    int first, apart;
    if constexpr (TYPE == JL_Q6_K) {
        const int h = j >> 3, i = j & 7;
        first = 128 * h + 32 * (i >> 2) + 8 * (i & 3);
        apart = 64;
    } else if constexpr (TYPE == JL_Q5_K) {
        first = 64 * (j >> 2) + 8 * (j & 3);
        apart = 32;
    } else {
        first = 32 * (j >> 1) + 8 * (j & 1);
        apart = 16;
    }
    const float4 *xs = (const float4 *)(x + first);
    v.x[0] = xs[0];
    v.x[1] = xs[1];
    v.x[2] = xs[apart / 4];
    v.x[3] = xs[apart / 4 + 1];
#pragma unroll
    for (int g = 0; g < 2; g++) {
        const float4 p = v.x[2 * g], q = v.x[2 * g + 1];
        const float sum = ((p.x + p.y) + (p.z + p.w)) + ((q.x + q.y) + (q.z + q.w));
        v.m32[g] = TYPE == JL_Q6_K ? -32.f * sum : TYPE == JL_Q5_0 ? -16.f * sum : TYPE == JL_IQ4_XS ? -128.f * sum : sum;
    }
    return v;
}

template <int TYPE>
__device__ __forceinline__ float block_part(const Raw<TYPE> &r, const Xs &v, int j) {
    if constexpr (TYPE == JL_Q6_K) {
        const int i = j & 7;
        const float d = jl_half_bits_to_float(r.d);
        const int sel = i >> 2;                    // 0: groups 0 and 2, 1: groups 1 and 3
        // bits 4-5 of the low-nibble group are qh >> 2 sel, of the high-nibble group qh >> (2 sel + 4)
        const uint32_t h0 = r.qh.lo >> (2 * sel), h1 = r.qh.hi >> (2 * sel);
        const uint32_t lo0 = (r.ql.lo & 0x0F0F0F0Fu) | ((h0 & 0x03030303u) << 4);
        const uint32_t lo1 = (r.ql.hi & 0x0F0F0F0Fu) | ((h1 & 0x03030303u) << 4);
        const uint32_t hi0 = ((r.ql.lo >> 4) & 0x0F0F0F0Fu) | (h0 & 0x30303030u);
        const uint32_t hi1 = ((r.ql.hi >> 4) & 0x0F0F0F0Fu) | (h1 & 0x30303030u);
        // scales: byte (position / 16) + 2 group of the half's eight; positions 8 (i & 3) .. + 7
        const int at = ((i & 3) >> 1) + 2 * sel;
        const uint64_t s8 = ((uint64_t)r.s8.hi << 32) | r.s8.lo;
        const float sc_lo = (float)(int)(int8_t)(s8 >> (8 * at));
        const float sc_hi = (float)(int)(int8_t)(s8 >> (8 * (at + 4)));
        const float lo = (dot4(lo0, v.x[0]) + dot4(lo1, v.x[1])) + v.m32[0];
        const float hi = (dot4(hi0, v.x[2]) + dot4(hi1, v.x[3])) + v.m32[1];
        return d * fmaf(sc_hi, hi, sc_lo * lo);
    } else if constexpr (TYPE == JL_Q4_1) {
        const float d = jl_half_bits_to_float(r.dm), m = jl_half_bits_to_float(r.dm >> 16);
        const float lo = dot4(r.qs.lo & 0x0F0F0F0Fu, v.x[0]) + dot4(r.qs.hi & 0x0F0F0F0Fu, v.x[1]);
        const float hi = dot4((r.qs.lo >> 4) & 0x0F0F0F0Fu, v.x[2]) + dot4((r.qs.hi >> 4) & 0x0F0F0F0Fu, v.x[3]);
        return fmaf(d, lo + hi, m * (v.m32[0] + v.m32[1]));
    } else if constexpr (TYPE == JL_Q5_0) {
        // fifth bits: byte `half` of qh for the low-nibble eight, byte 2 + half for the high-nibble eight
        const uint32_t bl = r.qh.v >> (8 * (j & 1)), bh = r.qh.v >> (16 + 8 * (j & 1));
        const uint32_t lo0 = (r.qs.lo & 0x0F0F0F0Fu) | (jl_spread4(bl) << 4);
        const uint32_t lo1 = (r.qs.hi & 0x0F0F0F0Fu) | (jl_spread4(bl >> 4) << 4);
        const uint32_t hi0 = ((r.qs.lo >> 4) & 0x0F0F0F0Fu) | (jl_spread4(bh) << 4);
        const uint32_t hi1 = ((r.qs.hi >> 4) & 0x0F0F0F0Fu) | (jl_spread4(bh >> 4) << 4);
        const float lo = (dot4(lo0, v.x[0]) + dot4(lo1, v.x[1])) + v.m32[0];
        const float hi = (dot4(hi0, v.x[2]) + dot4(hi1, v.x[3])) + v.m32[1];
        return jl_half_bits_to_float(r.d) * (lo + hi);
    } else if constexpr (TYPE == JL_IQ4_XS) {
        const int g = j >> 1;
        const uint32_t scales_h = r.hdr.x >> 16, scales_l = r.hdr.y;
        const int ls = (int)(((scales_l >> (4 * g)) & 0xFu) | (((scales_h >> (2 * g)) & 3u) << 4));
        const float dl = jl_half_bits_to_float(r.hdr.x) * (float)(ls - 32);
        // table values with 128 added are bytes 1..241; the 128 comes off through m32
        const uint32_t lo0 = jl_iq4nl_lookup4(r.qs.x & 0x0F0F0F0Fu) ^ 0x80808080u;
        const uint32_t lo1 = jl_iq4nl_lookup4(r.qs.y & 0x0F0F0F0Fu) ^ 0x80808080u;
        const uint32_t hi0 = jl_iq4nl_lookup4((r.qs.x >> 4) & 0x0F0F0F0Fu) ^ 0x80808080u;
        const uint32_t hi1 = jl_iq4nl_lookup4((r.qs.y >> 4) & 0x0F0F0F0Fu) ^ 0x80808080u;
        const float lo = (dot4(lo0, v.x[0]) + dot4(lo1, v.x[1])) + v.m32[0];
        const float hi = (dot4(hi0, v.x[2]) + dot4(hi1, v.x[3])) + v.m32[1];
        return dl * (lo + hi);
    } else {
        const int pair = j >> 2;
        const float d = jl_half_bits_to_float(r.hdr.x), dmin = jl_half_bits_to_float(r.hdr.x >> 16);
        // fifth bits: bit 2 pair of qh for the low-nibble sub-block, bit 2 pair + 1 for the high one
        const uint32_t b0 = r.qh.x >> (2 * pair), b1 = r.qh.y >> (2 * pair);
        const uint32_t lo0 = (r.qs.x & 0x0F0F0F0Fu) | ((b0 & 0x01010101u) << 4);
        const uint32_t lo1 = (r.qs.y & 0x0F0F0F0Fu) | ((b1 & 0x01010101u) << 4);
        const uint32_t hi0 = ((r.qs.x >> 4) & 0x0F0F0F0Fu) | ((b0 & 0x02020202u) << 3);
        const uint32_t hi1 = ((r.qs.y >> 4) & 0x0F0F0F0Fu) | ((b1 & 0x02020202u) << 3);
        int sc0, mn0, sc1, mn1;
        jl_q4k_scale_min(r.hdr.y, r.hdr.z, r.hdr.w, 2 * pair, sc0, mn0);
        jl_q4k_scale_min(r.hdr.y, r.hdr.z, r.hdr.w, 2 * pair + 1, sc1, mn1);
        const float lo = dot4(lo0, v.x[0]) + dot4(lo1, v.x[1]);
        const float hi = dot4(hi0, v.x[2]) + dot4(hi1, v.x[3]);
        const float scaled = fmaf((float)sc1, hi, (float)sc0 * lo);
        const float mins = fmaf((float)mn1, v.m32[1], (float)mn0 * v.m32[0]);
        return fmaf(d, scaled, -dmin * mins);
    }
}

template <int TYPE> struct Geometry;
template <> struct Geometry<JL_Q6_K> { static constexpr int kBytes = 210; };
template <> struct Geometry<JL_Q5_K> { static constexpr int kBytes = 176; };
// bytes per 256 elements: eight blocks of Q4_1 / Q5_0, one super-block of IQ4_XS
template <> struct Geometry<JL_Q4_1> { static constexpr int kBytes = 160; };
template <> struct Geometry<JL_Q5_0> { static constexpr int kBytes = 176; };
template <> struct Geometry<JL_IQ4_XS> { static constexpr int kBytes = 136; };

// DUAL: `w_up` is a second weight of the same shape and a row's result is SiLU(w . x) * (w_up . x),
// the fused gate/up of the feed-forward block (the reference fuses it for Q5_K,
// J/backend/tornado/layers/QuantizedProjections.java:386-393).
template <int TYPE, bool DUAL>
__global__ void __launch_bounds__(256)
jl_gemv_direct(const uint8_t *__restrict__ w, const uint8_t *__restrict__ w_up, const float *__restrict__ x,
               float *__restrict__ out, int rows, int n, int epilogue) {
    constexpr int BB = Geometry<TYPE>::kBytes;
    const int lane = threadIdx.x & 63;
    const int waves = (gridDim.x * blockDim.x) >> 6;
    const int blocks = n >> 8;                 // super-blocks per row
    const int j = lane & 15;
    for (int row = (blockIdx.x * blockDim.x + threadIdx.x) >> 6; row < rows; row += waves) {
        const uint8_t *wr = w + (int64_t)row * blocks * BB;
        const uint8_t *ur = DUAL ? w_up + (int64_t)row * blocks * BB : nullptr;
        float acc = 0.f, acc_up = 0.f;
        // two super-blocks per lane and trip: all their loads are issued before the first use
        for (int sb0 = lane >> 4; sb0 < blocks; sb0 += 8) {
            Raw<TYPE> r[2], ru[2];
            Xs v[2];
#pragma unroll
            for (int u = 0; u < 2; u++) {
                const int sb = sb0 + 4 * u;
                if (sb < blocks) {
                    r[u] = load_raw<TYPE>(wr + sb * BB, j);
                    if constexpr (DUAL) ru[u] = load_raw<TYPE>(ur + sb * BB, j);
                    v[u] = load_x<TYPE>(x + sb * 256, j);
                }
            }
#pragma unroll
            for (int u = 0; u < 2; u++)
                if (sb0 + 4 * u < blocks) {
                    acc += block_part<TYPE>(r[u], v[u], j);
                    if constexpr (DUAL) acc_up += block_part<TYPE>(ru[u], v[u], j);
                }
        }
        acc = jl_group_sum<JL_WAVE>(acc);
        if constexpr (DUAL) acc_up = jl_group_sum<JL_WAVE>(acc_up);
        if (lane == 0) {
            if constexpr (DUAL) out[row] = jl_swiglu_value(acc, acc_up);
            else if (epilogue == JL_RESIDUAL) out[row] += acc;
            else out[row] = acc;
        }
    }
}

// Rows of 4 NIT super-blocks: a lane meets the same activations in every row, so they are read
// once into registers, and a row's 6 NIT loads per lane are all in flight before the first use.
template <int TYPE, int NIT, bool DUAL>
__global__ void __launch_bounds__(256)
jl_gemv_direct_held(const uint8_t *__restrict__ w, const uint8_t *__restrict__ w_up, const float *__restrict__ x,
                    float *__restrict__ out, int rows, int epilogue) {
    constexpr int BB = Geometry<TYPE>::kBytes;
    const int lane = threadIdx.x & 63;
    const int waves = (gridDim.x * blockDim.x) >> 6;
    const int j = lane & 15;
    Xs v[NIT];
#pragma unroll
    for (int k = 0; k < NIT; k++) v[k] = load_x<TYPE>(x + ((lane >> 4) + 4 * k) * 256, j);
    for (int row = (blockIdx.x * blockDim.x + threadIdx.x) >> 6; row < rows; row += waves) {
        const int64_t at = (int64_t)row * (4 * NIT * BB) + (lane >> 4) * BB;
        Raw<TYPE> r[NIT];
#pragma unroll
        for (int k = 0; k < NIT; k++) r[k] = load_raw<TYPE>(w + at + k * 4 * BB, j);
        float acc = 0.f, acc_up = 0.f;
        if constexpr (DUAL) {
            // the up row's loads go out before the gate row is multiplied
            Raw<TYPE> ru[NIT];
#pragma unroll
            for (int k = 0; k < NIT; k++) ru[k] = load_raw<TYPE>(w_up + at + k * 4 * BB, j);
#pragma unroll
            for (int k = 0; k < NIT; k++) acc += block_part<TYPE>(r[k], v[k], j);
#pragma unroll
            for (int k = 0; k < NIT; k++) acc_up += block_part<TYPE>(ru[k], v[k], j);
            acc_up = jl_group_sum<JL_WAVE>(acc_up);
        } else {
#pragma unroll
            for (int k = 0; k < NIT; k++) acc += block_part<TYPE>(r[k], v[k], j);
        }
        acc = jl_group_sum<JL_WAVE>(acc);
        if (lane == 0) {
            if constexpr (DUAL) out[row] = jl_swiglu_value(acc, acc_up);
            else if (epilogue == JL_RESIDUAL) out[row] += acc;
            else out[row] = acc;
        }
    }
}

// J/tensor/standard/Q6_KFloatTensor.java:66-122, one thread per element: (d * scale) * (q - 32),
// each product rounded to fp32.
__global__ void __launch_bounds__(256)
jl_dequant_q6_k(const uint8_t *__restrict__ w, float *__restrict__ out, int64_t total) {
    const int64_t e = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (e >= total) return;
    const uint8_t *blk = w + (e >> 8) * 210;
    const int within = (int)(e & 255);
    const int h = within >> 7, group = (within >> 5) & 3, pos = within & 31;
    const int ql = blk[64 * h + 32 * (group & 1) + pos];
    const int qh = blk[128 + 32 * h + pos];
    const int low = (group >> 1) ? (ql >> 4) : (ql & 0xF);
    const int q = (low | (((qh >> (2 * group)) & 3) << 4)) - 32;
    const int sc = (int)(int8_t)blk[192 + 8 * h + (pos >> 4) + 2 * group];
    const float d = jl_half_bits_to_float(blk[208] | (blk[209] << 8));
    out[e] = jl_mul_rn(jl_mul_rn(d, (float)sc), (float)q);
}

// J/tensor/standard/Q5_KFloatTensor.java:78-122, one thread per element: ((d * sc) * q) - (dmin * m),
// every product and the difference rounded to fp32.
__global__ void __launch_bounds__(256)
jl_dequant_q5_k(const uint8_t *__restrict__ w, float *__restrict__ out, int64_t total) {
    const int64_t e = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (e >= total) return;
    const uint8_t *blk = w + (e >> 8) * 176;
    const uint32_t *hdr = (const uint32_t *)blk;
    const float d = jl_half_bits_to_float(hdr[0]), dmin = jl_half_bits_to_float(hdr[0] >> 16);
    const int within = (int)(e & 255);
    const int pair = within >> 6, high = (within >> 5) & 1, pos = within & 31;
    const int byte = blk[48 + 32 * pair + pos];
    int q = high ? (byte >> 4) : (byte & 0xF);
    q += ((blk[16 + pos] >> (2 * pair + high)) & 1) * 16;
    int sc, mn;
    jl_q4k_scale_min(hdr[1], hdr[2], hdr[3], 2 * pair + high, sc, mn);
    float t = jl_mul_rn(d, (float)sc);
    t = jl_mul_rn(t, (float)q);
    out[e] = __fsub_rn(t, jl_mul_rn(dmin, (float)mn));
}

// J/tensor/standard/Q4_1FloatTensor.java:73-94: (nibble * d) + m, Q5_0FloatTensor.java:61-85:
// d * (q - 16), IQ4_XSFloatTensor.java:72-100: (d * (ls - 32)) * kvalues[q]; one thread per element,
// every operation rounded to fp32.
template <int TYPE>
__global__ void __launch_bounds__(256)
jl_dequant_nibbles(const uint8_t *__restrict__ w, float *__restrict__ out, int64_t total) {
    const int64_t e = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (e >= total) return;
    const int within = (int)(e & 31);       // position in the group of 32
    const int byte_at = within & 15, shift = (within >> 4) * 4;
    if constexpr (TYPE == JL_Q4_1) {
        const uint8_t *blk = w + (e >> 5) * 20;
        const uint32_t dm = *(const uint32_t *)blk;
        const int q = (blk[4 + byte_at] >> shift) & 0xF;
        out[e] = __fadd_rn(jl_mul_rn((float)q, jl_half_bits_to_float(dm)), jl_half_bits_to_float(dm >> 16));
    } else if constexpr (TYPE == JL_Q5_0) {
        const uint8_t *blk = w + (e >> 5) * 22;
        const uint32_t qh = blk[2] | (blk[3] << 8) | (blk[4] << 16) | ((uint32_t)blk[5] << 24);
        const int q = ((blk[6 + byte_at] >> shift) & 0xF) | (int)(((qh >> within) & 1u) << 4);
        out[e] = jl_mul_rn(jl_half_bits_to_float(blk[0] | (blk[1] << 8)), (float)(q - 16));
    } else {
        const uint8_t *blk = w + (e >> 8) * 136;
        const int g = (int)((e >> 5) & 7);
        const uint2 hdr = *(const uint2 *)blk;
        const int ls = (int)(((hdr.y >> (4 * g)) & 0xFu) | ((((hdr.x >> 16) >> (2 * g)) & 3u) << 4));
        const float dl = jl_mul_rn(jl_half_bits_to_float(hdr.x), (float)(ls - 32));
        const uint32_t q = (blk[8 + 16 * g + byte_at] >> shift) & 0xFu;
        const int kv = (int)(int8_t)(jl_iq4nl_lookup4(q) & 0xFFu);
        out[e] = jl_mul_rn(dl, (float)kv);
    }
}

template <int TYPE, bool DUAL>
int launch_direct(jl_context *ctx, const jl_weight *w, const jl_weight *w_up, const float *x, float *out, int epilogue) {
    const int rows = (int)w->rows, n = (int)w->cols;
    const uint8_t *up = DUAL ? w_up->blocks : nullptr;
    // enough waves to hide the loads' latency, rows dealt round robin
    int groups = (rows + 3) / 4;
    const int cap = ctx->compute_units * 8;
    if (groups > cap) groups = cap;
    const dim3 g(groups), b(256);
    // (a gate/up pair holds twice the raw registers: rows of 8192 columns take the general kernel)
    switch (n) {
        case 1024: hipLaunchKernelGGL((jl_gemv_direct_held<TYPE, 1, DUAL>), g, b, 0, ctx->stream, w->blocks, up, x, out, rows, epilogue); break;
        case 2048: hipLaunchKernelGGL((jl_gemv_direct_held<TYPE, 2, DUAL>), g, b, 0, ctx->stream, w->blocks, up, x, out, rows, epilogue); break;
        case 4096: hipLaunchKernelGGL((jl_gemv_direct_held<TYPE, 4, DUAL>), g, b, 0, ctx->stream, w->blocks, up, x, out, rows, epilogue); break;
        case 8192:
            if constexpr (!DUAL) {
                hipLaunchKernelGGL((jl_gemv_direct_held<TYPE, 8, false>), g, b, 0, ctx->stream, w->blocks, up, x, out, rows, epilogue);
                break;
            }
            [[fallthrough]];
        default: hipLaunchKernelGGL((jl_gemv_direct<TYPE, DUAL>), g, b, 0, ctx->stream, w->blocks, up, x, out, rows, n, epilogue); break;
    }
    JL_HIP(hipGetLastError());
    return JL_OK;
}

template <int TYPE>
int launch_direct_type(jl_context *ctx, const jl_weight *w, const jl_weight *w_up, const float *x, float *out, int epilogue) {
    return w_up ? launch_direct<TYPE, true>(ctx, w, w_up, x, out, epilogue)
                : launch_direct<TYPE, false>(ctx, w, nullptr, x, out, epilogue);
}

}  // namespace

int jl_launch_gemv_direct(jl_context *ctx, const jl_weight *w, const jl_weight *w_up, const float *x, float *out,
                          int epilogue) {
    if (w->cols % 256 != 0 || ((uintptr_t)x & 15) != 0) {
        return jl_fail(JL_ERR_UNSUPPORTED, "no %s projection kernel for a row length of %lld or an unaligned vector",
                       jl_type_name(w->type), (long long)w->cols);
    }
    switch (w->type) {
        case JL_Q6_K: return launch_direct_type<JL_Q6_K>(ctx, w, w_up, x, out, epilogue);
        case JL_Q5_K: return launch_direct_type<JL_Q5_K>(ctx, w, w_up, x, out, epilogue);
        case JL_Q4_1: return launch_direct_type<JL_Q4_1>(ctx, w, w_up, x, out, epilogue);
        case JL_Q5_0: return launch_direct_type<JL_Q5_0>(ctx, w, w_up, x, out, epilogue);
        case JL_IQ4_XS: return launch_direct_type<JL_IQ4_XS>(ctx, w, w_up, x, out, epilogue);
        default: return jl_fail(JL_ERR_UNSUPPORTED, "no projection kernel for a ggml type %d weight", w->type);
    }
}

int jl_launch_dequant_direct(jl_context *ctx, const jl_weight *w, float *out) {
    const int64_t total = w->rows * w->cols;
    const dim3 g((unsigned)((total + 255) / 256)), b(256);
    switch (w->type) {
        case JL_Q6_K: hipLaunchKernelGGL(jl_dequant_q6_k, g, b, 0, ctx->stream, w->blocks, out, total); break;
        case JL_Q5_K: hipLaunchKernelGGL(jl_dequant_q5_k, g, b, 0, ctx->stream, w->blocks, out, total); break;
        case JL_Q4_1: hipLaunchKernelGGL(jl_dequant_nibbles<JL_Q4_1>, g, b, 0, ctx->stream, w->blocks, out, total); break;
        case JL_Q5_0: hipLaunchKernelGGL(jl_dequant_nibbles<JL_Q5_0>, g, b, 0, ctx->stream, w->blocks, out, total); break;
        case JL_IQ4_XS: hipLaunchKernelGGL(jl_dequant_nibbles<JL_IQ4_XS>, g, b, 0, ctx->stream, w->blocks, out, total); break;
        default: return jl_fail(JL_ERR_UNSUPPORTED, "jl_dequant_f32: no decode kernel for ggml type %d", w->type);
    }
    JL_HIP(hipGetLastError());
    return JL_OK;
}
