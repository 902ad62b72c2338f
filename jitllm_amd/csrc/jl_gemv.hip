// Decode matrix-vector kernels for Q8_0 / Q4_0 / Q4_K weights in their GGUF block layout.
//
// Replaces the one-workgroup-per-row TornadoVM kernels of the reference
// (J/backend/tornado/kernels/TransformerComputeKernelsLayered.java:2222-2479,
//  TransformerComputeKernelsQ4_0.java:531-701, TransformerComputeKernelsQ4_K.java:673-842)
// with a tile-streaming design for CDNA4:
//
//   * a thread owns one 64-element column slice of the row for the whole kernel and keeps those 64
//     activations in registers (loaded once, through LDS, coalesced);
//   * a workgroup walks tiles of R consecutive rows.  A tile is one contiguous byte range of the
//     weight (R * row_bytes), copied global -> registers -> LDS with 128-bit loads that ignore
//     block boundaries, so the 34- and 18-byte block strides never reach the memory system;
//   * each thread then reads its own slice of the tile from LDS with 32-bit reads -- a slice is a
//     pair of Q8_0 blocks (68 B), a pair of Q4_0 blocks (36 B) or a quarter of a Q4_K super-block
//     (32 B of nibbles + the shared 16 B header), all 4-byte aligned -- and unpacks in registers;
//   * the next tile's global loads are in flight while the current tile is computed (two LDS
//     stages, one barrier per tile);
//   * row sums fold across lanes with wave shuffles, and across waves (rows wider than 4096
//     columns) through a few LDS words.
//
// Memory-bound by design: no MFMA here.  Summation order differs from the host's sequential or
// lane-wise order, so results are held to a tolerance, not to bit equality; the element decode
// itself is held bit-equal by the kernels in jl_dequant.hip.
#include "jl_device.h"
#include "jl_internal.h"

#include <climits>
#include <map>
#include <mutex>
#include <tuple>

namespace {

constexpr int kMaxSeg = 3;

struct GemvParams {
    const uint8_t *w[kMaxSeg];   // weight of each segment (q | k | v, or a single projection)
    float *out[kMaxSeg];
    int seg_rows[kMaxSeg];
    int seg_tile_begin[kMaxSeg + 1];  // first tile of each segment; [nseg] = total tiles
    int nseg;
    const uint8_t *w_up;  // JL_SWIGLU: the up weight, same shape as w[0]
    const float *x;
    int n;          // row length
    int S;          // 64-element slices per row
    int Sp;         // S padded to the next power of two
    int R;          // rows per tile
    int row_bytes;
    int epilogue;
    // RMS normalisation folded into the activation load: x_j becomes rms_w[j] * (scale * x_j).
    const float *rms_w;      // null: x is used as it is
    const float *rms_scale;  // device scalar; null with rms_w set: the kernel computes
                             // 1 / sqrt(sum x^2 / n + rms_eps) itself, every workgroup for itself
    float rms_eps;
    // Packed-integer mode: the activation as Q8 blocks (32 signed bytes, an fp32 scale and the sum
    // of the bytes per block) instead of x.
    const int8_t *xq;
    const float *xq_scales;
    const int32_t *xq_sums;
    // The ARGMAX instances leave every workgroup's largest output, and its row, in cell blockIdx.x.
    float *best_value;
    int *best_index;
};

// Bytes of a tile a thread brings in: kX4 sixteen-byte loads and kTail four-byte ones.  For the
// three main types that is exactly a thread's 64-column slice, so every load slot is real data; a
// Q6_K slice is 52.5 bytes (210 per 256 columns), its threads bring in 64 each and the slots past
// the tile's end re-read a dummy address.
template <int TYPE> struct Traits;
template <> struct Traits<JL_Q8_0> { static constexpr int kX4 = 4, kTail = 1; };  // 68 B = 4 x 16 + 4
template <> struct Traits<JL_Q4_0> { static constexpr int kX4 = 2, kTail = 1; };  // 36 B = 2 x 16 + 4
template <> struct Traits<JL_Q4_K> { static constexpr int kX4 = 2, kTail = 1; };  // 144 B / 4 = 36 B
template <> struct Traits<JL_Q6_K> { static constexpr int kX4 = 4, kTail = 0; };  // 64 B >= 210 B / 4
template <> struct Traits<JL_Q5_K> { static constexpr int kX4 = 3, kTail = 0; };  // 48 B >= 176 B / 4
template <> struct Traits<JL_Q4_1> { static constexpr int kX4 = 3, kTail = 0; };  // 48 B >= 2 x 20 B
template <> struct Traits<JL_Q5_0> { static constexpr int kX4 = 3, kTail = 0; };  // 48 B >= 2 x 22 B
template <> struct Traits<JL_IQ4_XS> { static constexpr int kX4 = 3, kTail = 0; };  // 48 B >= 136 B / 4
// the three types every entry point exists for; the others have the plain, residual and gate/up forms
constexpr bool is_main_type(int type) { return type == JL_Q8_0 || type == JL_Q4_0 || type == JL_Q4_K; }
// the others the tile kernel takes
constexpr bool is_side_type(int type) {
    return type == JL_Q6_K || type == JL_Q5_K || type == JL_Q4_1 || type == JL_Q5_0 || type == JL_IQ4_XS;
}
// bytes of a row of `slices` 64-column slices
template <int TYPE>
__device__ __host__ constexpr int row_bytes_of(int slices) {
    return TYPE == JL_Q8_0 ? slices * 68 : TYPE == JL_Q6_K ? slices / 4 * 210 : TYPE == JL_Q5_K ? slices * 44
           : TYPE == JL_Q4_1 ? slices * 40 : TYPE == JL_Q5_0 ? slices * 44 : TYPE == JL_IQ4_XS ? slices * 34 : slices * 36;
}

__device__ __forceinline__ float ubyte(uint32_t v, int k) { return (float)((v >> (8 * k)) & 0xFFu); }
__device__ __forceinline__ float sbyte(uint32_t v, int k) { return (float)(int)(int8_t)(v >> (8 * k)); }

// Dot of one Q8_0 block pair (68 bytes, 4-byte aligned in LDS) with 64 activations.
//   bytes 0..1 scale A | 2..33 quants A | 34..35 scale B | 36..67 quants B
__device__ __forceinline__ float slice_dot_q8_0(const uint32_t (&w)[17], const float (&x)[64]) {
    float dA = jl_half_bits_to_float(w[0]);
    float dB = jl_half_bits_to_float(w[8] >> 16);
    float a0 = 0.f, a1 = 0.f, b0 = 0.f, b1 = 0.f;
    // block A: element i sits at byte 2 + i of the slice
#pragma unroll
    for (int i = 0; i < 32; i++) {
        int o = 2 + i;
        float q = sbyte(w[o >> 2], o & 3);
        if (i & 1) a1 = fmaf(q, x[i], a1); else a0 = fmaf(q, x[i], a0);
    }
    // block B: element i sits at byte 36 + i
#pragma unroll
    for (int i = 0; i < 32; i++) {
        float q = sbyte(w[9 + (i >> 2)], i & 3);
        if (i & 1) b1 = fmaf(q, x[32 + i], b1); else b0 = fmaf(q, x[32 + i], b0);
    }
    return fmaf(a0 + a1, dA, (b0 + b1) * dB);
}

// The 4-bit kernels multiply without converting: a nibble left alone in the low ten bits of a
// 16-bit half *is* a binary16 number -- the subnormal q * 2^-24 (q * 2^-20 for a high nibble, which
// sits four bits up) -- and v_fma_mix_f32 takes a binary16 operand from either half of a register,
// widens it exactly and fuses product and sum in fp32.  So a dword of eight nibbles costs five
// mask / shift operations and eight multiply-adds, where byte -> float conversions took sixteen
// more; the powers of two are taken out again, exactly, with the block scale.
struct NibblePairs {
    uint32_t lo02, hi02, lo13, hi13;   // low / high nibbles of bytes 0 and 2, of bytes 1 and 3
};
__device__ __forceinline__ NibblePairs nibble_pairs(uint32_t v) {
    const uint32_t t = v >> 8;
    return NibblePairs{v & 0x000F000Fu, v & 0x00F000F0u, t & 0x000F000Fu, t & 0x00F000F0u};
}
// acc += (binary16 in the low / high half of w) * x
__device__ __forceinline__ void mix_low(float &acc, uint32_t w, float x) {
    asm("v_fma_mix_f32 %0, %1, %2, %0 op_sel:[0,0,0] op_sel_hi:[1,0,0]" : "+v"(acc) : "v"(w), "v"(x));
}
__device__ __forceinline__ void mix_high(float &acc, uint32_t w, float x) {
    asm("v_fma_mix_f32 %0, %1, %2, %0 op_sel:[1,0,0] op_sel_hi:[1,0,0]" : "+v"(acc) : "v"(w), "v"(x));
}
// byte b (0..3) of the dword the pairs came from: acc_lo += low nibble * 2^-24 * x_lo,
// acc_hi += high nibble * 2^-20 * x_hi
__device__ __forceinline__ void mix_byte(const NibblePairs &n, int b, float x_lo, float x_hi, float &acc_lo,
                                         float &acc_hi) {
    const uint32_t lo = (b & 1) ? n.lo13 : n.lo02, hi = (b & 1) ? n.hi13 : n.hi02;
    if (b & 2) {
        mix_high(acc_lo, lo, x_lo);
        mix_high(acc_hi, hi, x_hi);
    } else {
        mix_low(acc_lo, lo, x_lo);
        mix_low(acc_hi, hi, x_hi);
    }
}
constexpr float kTwo24 = 16777216.f, kTwoM24 = 1.f / 16777216.f;

// Dot of one Q4_0 block pair (36 bytes) with 64 activations; sx[0], sx[1] are the sums of the
// activations facing block A and block B, so that sum((q - 8) x) = sum(q x) - 8 sum(x).
//   bytes 0..1 scale A | 2..17 nibbles A | 18..19 scale B | 20..35 nibbles B
// element i < 16 of a block is the low nibble of its byte i, element 16 + i the high nibble.
__device__ __forceinline__ float slice_dot_q4_0(const uint32_t (&dw)[9], const float (&x)[64],
                                                const float (&sx)[4]) {
    NibblePairs n[9];
#pragma unroll
    for (int i = 0; i < 9; i++) n[i] = nibble_pairs(dw[i]);
    const float dA = jl_half_bits_to_float(dw[0]);
    const float dB = jl_half_bits_to_float(dw[4] >> 16);
    // a0, b0: sum(q x) * 2^-24 over the low nibbles; a1, b1: * 2^-20 over the high nibbles
    float a0 = 0.f, a1 = 0.f, b0 = 0.f, b1 = 0.f;
#pragma unroll
    for (int i = 0; i < 16; i++) {
        const int o = 2 + i;  // byte i of block A
        mix_byte(n[o >> 2], o & 3, x[i], x[16 + i], a0, a1);
    }
#pragma unroll
    for (int i = 0; i < 16; i++) {
        const int o = 20 + i;  // byte i of block B
        mix_byte(n[o >> 2], o & 3, x[32 + i], x[48 + i], b0, b1);
    }
    const float da = fmaf(-8.f * kTwoM24, sx[0], fmaf(a1, 0.0625f, a0));
    const float db = fmaf(-8.f * kTwoM24, sx[1], fmaf(b1, 0.0625f, b0));
    return fmaf(da, dA * kTwo24, db * (dB * kTwo24));
}

// Dot of one quarter of a Q4_K super-block with 64 activations.  `hdr` is the super-block's first
// 16 bytes (d, dmin, 12 packed scale bytes), `qs` the 32 nibble bytes of pair `pair`: low nibbles
// are sub-block 2*pair (activations 0..31), high nibbles sub-block 2*pair+1 (activations 32..63).
// sum(w x) = (d sc) sum(q x) - (dmin m) sum(x) per sub-block.
__device__ __forceinline__ float slice_dot_q4_k(const uint4 &h, const uint4 &q0, const uint4 &q1,
                                                int pair, const float (&x)[64],
                                                const float (&sx)[4]) {
    const uint32_t w[8] = {q0.x, q0.y, q0.z, q0.w, q1.x, q1.y, q1.z, q1.w};
    const float d = jl_half_bits_to_float(h.x);
    const float dmin = jl_half_bits_to_float(h.x >> 16);
    int sc0, mn0, sc1, mn1;
    jl_q4k_scale_min(h.y, h.z, h.w, 2 * pair, sc0, mn0);
    jl_q4k_scale_min(h.y, h.z, h.w, 2 * pair + 1, sc1, mn1);
    // a: sum(q x) * 2^-24 of the low sub-block, b: * 2^-20 of the high one; even and odd bytes apart
    float a0 = 0.f, a1 = 0.f, b0 = 0.f, b1 = 0.f;
#pragma unroll
    for (int i = 0; i < 8; i++) {
        const NibblePairs n = nibble_pairs(w[i]);
        mix_byte(n, 0, x[4 * i + 0], x[32 + 4 * i + 0], a0, b0);
        mix_byte(n, 1, x[4 * i + 1], x[32 + 4 * i + 1], a1, b1);
        mix_byte(n, 2, x[4 * i + 2], x[32 + 4 * i + 2], a0, b0);
        mix_byte(n, 3, x[4 * i + 3], x[32 + 4 * i + 3], a1, b1);
    }
    float lo_term = ((d * (float)sc0) * kTwo24) * (a0 + a1) - (dmin * (float)mn0) * sx[0];
    float hi_term = ((d * (float)sc1) * (kTwo24 * 0.0625f)) * (b0 + b1) - (dmin * (float)mn1) * sx[1];
    return lo_term + hi_term;
}

// acc += (the four bytes of v, values up to 255, as binary16 subnormals b * 2^-24) . x[0..3]
__device__ __forceinline__ void mix_bytes4(float &acc, uint32_t v, float x0, float x1, float x2, float x3) {
    const uint32_t even = v & 0x00FF00FFu, odd = (v >> 8) & 0x00FF00FFu;
    mix_low(acc, even, x0);
    mix_low(acc, odd, x1);
    mix_high(acc, even, x2);
    mix_high(acc, odd, x3);
}

// Dot of a quarter of a Q6_K super-block (ql[128] | qh[64] | 16 signed scales | fp16 d,
// J/tensor/standard/Q6_KFloatTensor.java:66-122) with 64 activations.  Quarter (h, upper): the
// 64 ql bytes and 32 qh bytes of half h; element l < 32 of the quarter is nibble `upper` of ql[l]
// with bits 4 upper .. 4 upper + 1 of qh[l] on top, element 32 + l nibble `upper` of ql[32 + l]
// with bits 4 upper + 2 .. + 3 of qh[l].  w = d * scale * (q - 32) with one scale per 16 elements;
// sx are the sums of the activations facing each 16.
__device__ __forceinline__ float slice_dot_q6_k(const uint32_t (&ql)[16], const uint32_t (&qh)[8], uint32_t scales,
                                                uint32_t dbits, int upper, const float (&x)[64],
                                                const float (&sx)[4]) {
    const int shl = 4 * upper;
    float a[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int j = 0; j < 8; j++) {
        const uint32_t h = qh[j] >> shl;
        const uint32_t v0 = ((ql[j] >> shl) & 0x0F0F0F0Fu) | ((h & 0x03030303u) << 4);
        const uint32_t v1 = ((ql[8 + j] >> shl) & 0x0F0F0F0Fu) | ((h & 0x0C0C0C0Cu) << 2);
        mix_bytes4(a[j >> 2], v0, x[4 * j], x[4 * j + 1], x[4 * j + 2], x[4 * j + 3]);
        mix_bytes4(a[2 + (j >> 2)], v1, x[32 + 4 * j], x[32 + 4 * j + 1], x[32 + 4 * j + 2], x[32 + 4 * j + 3]);
    }
    const float d = jl_half_bits_to_float(dbits) * kTwo24;
    float acc = 0.f;
#pragma unroll
    for (int g = 0; g < 4; g++) {
        const float sc = (float)(int)(int8_t)(scales >> (8 * g));
        acc = fmaf(sc, fmaf(-32.f * kTwoM24, sx[g], a[g]), acc);
    }
    return acc * d;
}

// Dot of one Q4_1 block pair (40 bytes: fp16 d, m | 16 nibble bytes, twice;
// J/tensor/standard/Q4_1FloatTensor.java:73-94) with 64 activations: w = d q + m, so
// sum(w x) = d sum(q x) + m sum(x) per block.  Element i < 16 of a block is the low nibble of its
// byte i, element 16 + i the high nibble.
__device__ __forceinline__ float slice_dot_q4_1(const uint32_t (&dw)[10], const float (&x)[64],
                                                const float (&sx)[4]) {
    float acc = 0.f;
#pragma unroll
    for (int blk = 0; blk < 2; blk++) {
        const float d = jl_half_bits_to_float(dw[5 * blk]), m = jl_half_bits_to_float(dw[5 * blk] >> 16);
        float lo = 0.f, hi = 0.f;
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const NibblePairs n = nibble_pairs(dw[5 * blk + 1 + j]);
#pragma unroll
            for (int b = 0; b < 4; b++) mix_byte(n, b, x[32 * blk + 4 * j + b], x[32 * blk + 16 + 4 * j + b], lo, hi);
        }
        acc = fmaf(d * kTwo24, fmaf(hi, 0.0625f, lo), fmaf(m, sx[blk], acc));
    }
    return acc;
}

// Dot of one Q5_0 block pair (44 bytes: fp16 d | 32 fifth bits | 16 nibble bytes, twice;
// J/tensor/standard/Q5_0FloatTensor.java:61-85) with 64 activations: w = d (q - 16), q the nibble
// with its fifth bit on top; bit i of the 32 belongs to element i.  `qh`, `qs`: the fifth bits and
// the four nibble dwords of block A, then of block B.
__device__ __forceinline__ float slice_dot_q5_0(uint32_t dA, uint32_t dB, const uint32_t (&qh)[2],
                                                const uint32_t (&qs)[8], const float (&x)[64],
                                                const float (&sx)[4]) {
    float acc = 0.f;
#pragma unroll
    for (int blk = 0; blk < 2; blk++) {
        float lo = 0.f, hi = 0.f;
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const uint32_t q = qs[4 * blk + j];
            // elements 4 j .. 4 j + 3 (low nibbles, fifth bits 4 j ..) and 16 + 4 j .. (high nibbles)
            const uint32_t v0 = (q & 0x0F0F0F0Fu) | (jl_spread4(qh[blk] >> (4 * j)) << 4);
            const uint32_t v1 = ((q >> 4) & 0x0F0F0F0Fu) | (jl_spread4(qh[blk] >> (16 + 4 * j)) << 4);
            mix_bytes4(lo, v0, x[32 * blk + 4 * j], x[32 * blk + 4 * j + 1], x[32 * blk + 4 * j + 2], x[32 * blk + 4 * j + 3]);
            mix_bytes4(hi, v1, x[32 * blk + 16 + 4 * j], x[32 * blk + 16 + 4 * j + 1], x[32 * blk + 16 + 4 * j + 2],
                       x[32 * blk + 16 + 4 * j + 3]);
        }
        const float d = jl_half_bits_to_float(blk ? dB : dA);
        acc = fmaf(d * kTwo24, fmaf(-16.f * kTwoM24, sx[blk], lo + hi), acc);
    }
    return acc;
}

// Dot of a quarter of an IQ4_XS super-block (fp16 d | scales_h | scales_l[4] | qs[128];
// J/tensor/standard/IQ4_XSFloatTensor.java:72-100) with 64 activations: sub-blocks 2 q and 2 q + 1,
// w = d (ls - 32) kvalues_iq4nl[nibble] with a 6-bit ls per sub-block; the 16 nibble bytes of a
// sub-block hold elements 0..15 in their low halves and 16..31 in their high halves.  The table is
// used with 128 added (bytes 1..241), which comes off through the activations' sums.
__device__ __forceinline__ float slice_dot_iq4_xs(uint2 hdr, const uint32_t (&qs)[8], int q, const float (&x)[64],
                                                  const float (&sx)[4]) {
    const float d = jl_half_bits_to_float(hdr.x);
    const uint32_t scales_h = hdr.x >> 16, scales_l = hdr.y;
    float acc = 0.f;
#pragma unroll
    for (int sub = 0; sub < 2; sub++) {
        const int g = 2 * q + sub;
        const int ls = (int)(((scales_l >> (4 * g)) & 0xFu) | (((scales_h >> (2 * g)) & 3u) << 4));
        float lo = 0.f, hi = 0.f;
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const uint32_t w = qs[4 * sub + j];
            const uint32_t v0 = jl_iq4nl_lookup4(w & 0x0F0F0F0Fu) ^ 0x80808080u;
            const uint32_t v1 = jl_iq4nl_lookup4((w >> 4) & 0x0F0F0F0Fu) ^ 0x80808080u;
            mix_bytes4(lo, v0, x[32 * sub + 4 * j], x[32 * sub + 4 * j + 1], x[32 * sub + 4 * j + 2], x[32 * sub + 4 * j + 3]);
            mix_bytes4(hi, v1, x[32 * sub + 16 + 4 * j], x[32 * sub + 16 + 4 * j + 1], x[32 * sub + 16 + 4 * j + 2],
                       x[32 * sub + 16 + 4 * j + 3]);
        }
        acc = fmaf((d * (float)(ls - 32)) * kTwo24, fmaf(-128.f * kTwoM24, sx[sub], lo + hi), acc);
    }
    return acc;
}

// Dot of a quarter of a Q5_K super-block (fp16 d, dmin | 12 packed scale / min bytes | qh[32] |
// qs[128], J/tensor/standard/Q5_KFloatTensor.java:78-122) with 64 activations: Q4_K's layout with a
// fifth bit per weight -- bit 2 pair of qh[l] for the low-nibble sub-block, bit 2 pair + 1 for the
// high-nibble one.  sum(w x) = (d sc) sum(q x) - (dmin m) sum(x) per sub-block.
__device__ __forceinline__ float slice_dot_q5_k(const uint4 &h, const uint32_t (&qs)[8], const uint32_t (&qh)[8],
                                                int pair, const float (&x)[64], const float (&sx)[4]) {
    const float d = jl_half_bits_to_float(h.x);
    const float dmin = jl_half_bits_to_float(h.x >> 16);
    int sc0, mn0, sc1, mn1;
    jl_q4k_scale_min(h.y, h.z, h.w, 2 * pair, sc0, mn0);
    jl_q4k_scale_min(h.y, h.z, h.w, 2 * pair + 1, sc1, mn1);
    float a0 = 0.f, a1 = 0.f, b0 = 0.f, b1 = 0.f;
#pragma unroll
    for (int j = 0; j < 8; j++) {
        const uint32_t hb = qh[j] >> (2 * pair);
        const uint32_t v0 = (qs[j] & 0x0F0F0F0Fu) | ((hb & 0x01010101u) << 4);
        const uint32_t v1 = ((qs[j] >> 4) & 0x0F0F0F0Fu) | ((hb & 0x02020202u) << 3);
        mix_bytes4((j & 1) ? a1 : a0, v0, x[4 * j], x[4 * j + 1], x[4 * j + 2], x[4 * j + 3]);
        mix_bytes4((j & 1) ? b1 : b0, v1, x[32 + 4 * j], x[32 + 4 * j + 1], x[32 + 4 * j + 2], x[32 + 4 * j + 3]);
    }
    float lo_term = ((d * (float)sc0) * kTwo24) * (a0 + a1) - (dmin * (float)mn0) * sx[0];
    float hi_term = ((d * (float)sc1) * kTwo24) * (b0 + b1) - (dmin * (float)mn1) * sx[1];
    return lo_term + hi_term;
}

// ---- packed-integer mode -----------------------------------------------------------------------
//
// The reference's dp4a kernels (TransformerComputeKernelsQ8_0DP4A.java:35-68,
// TransformerComputeKernelsQ4_0.java:466-510, TransformerComputeKernelsQ4_K.java:599-668): the
// activation arrives quantised to Q8 blocks, a block's products are summed exactly in int32 by
// four-byte dot instructions and the two scales are applied to the block's sum.  A thread keeps its
// slice's 64 activation bytes in registers in the byte positions of the weights they meet, so the
// raw LDS words feed the dot instruction unshifted; positions that hold a weight scale face zeros.

struct PackedX {
    uint32_t q[18];   // Q8_0: A 0..8, B 9..16 | Q4_0: A low 0..4, A high 5..9, B low 10..13, B high 14..17
                      // | Q4_K: elements 0..31 in 0..7, 32..63 in 8..15
    float scale[2];
    float sum[2];     // the blocks' byte sums, as floats (|sum| <= 32 * 127)
};

__device__ __forceinline__ int dot4(uint32_t a, uint32_t b, int c) {
    return __builtin_amdgcn_sdot4((int)a, (int)b, c, false);
}

// xa: the eight dwords of a block's 32 activation bytes.  The block's weights start two bytes into
// their first dword (after the fp16 scale), so the bytes move up by two: nine dwords for 32 bytes
// (Q8_0), five for each half of 16 (Q4_0).
template <int N>
__device__ __forceinline__ void shift_two_bytes(const uint32_t *xa, uint32_t *out) {
    out[0] = xa[0] << 16;
#pragma unroll
    for (int i = 1; i < N; i++) out[i] = __builtin_amdgcn_alignbyte(xa[i], xa[i - 1], 2);
    out[N] = xa[N - 1] >> 16;
}

template <int TYPE>
__device__ __forceinline__ void pack_x(const uint32_t (&raw)[16], PackedX &x) {
    if constexpr (TYPE == JL_Q8_0) {
        shift_two_bytes<8>(&raw[0], &x.q[0]);
#pragma unroll
        for (int i = 0; i < 8; i++) x.q[9 + i] = raw[8 + i];
        x.q[17] = 0;
    } else if constexpr (TYPE == JL_Q4_0) {
        shift_two_bytes<4>(&raw[0], &x.q[0]);    // elements 0..15 of block A face the low nibbles
        shift_two_bytes<4>(&raw[4], &x.q[5]);    // elements 16..31 the high nibbles
#pragma unroll
        for (int i = 0; i < 8; i++) x.q[10 + i] = raw[8 + i];   // block B's nibble bytes are dword aligned
    } else {
#pragma unroll
        for (int i = 0; i < 16; i++) x.q[i] = raw[i];
        x.q[16] = x.q[17] = 0;
    }
}

// (weightScale * xScale) * dot per block (TransformerComputeKernelsQ8_0DP4A.java:58-66)
__device__ __forceinline__ float slice_dot_packed_q8_0(const uint32_t (&w)[17], const PackedX &x) {
    int da = 0, db = 0;
#pragma unroll
    for (int i = 0; i < 9; i++) da = dot4(w[i], x.q[i], da);
#pragma unroll
    for (int i = 0; i < 8; i++) db = dot4(w[9 + i], x.q[9 + i], db);
    const float sa = jl_half_bits_to_float(w[0]) * x.scale[0];
    const float sb = jl_half_bits_to_float(w[8] >> 16) * x.scale[1];
    return fmaf(sa, (float)da, sb * (float)db);
}

// weightScale * xScale * (dot - 8 * xSum) per block (TransformerComputeKernelsQ4_0.java:487-506)
__device__ __forceinline__ float slice_dot_packed_q4_0(const uint32_t (&w)[9], const PackedX &x) {
    int da = 0, db = 0;
#pragma unroll
    for (int i = 0; i < 5; i++) {
        da = dot4(w[i] & 0x0F0F0F0Fu, x.q[i], da);
        da = dot4((w[i] >> 4) & 0x0F0F0F0Fu, x.q[5 + i], da);
    }
#pragma unroll
    for (int i = 0; i < 4; i++) {
        db = dot4(w[5 + i] & 0x0F0F0F0Fu, x.q[10 + i], db);
        db = dot4((w[5 + i] >> 4) & 0x0F0F0F0Fu, x.q[14 + i], db);
    }
    const float sa = jl_half_bits_to_float(w[0]) * x.scale[0];
    const float sb = jl_half_bits_to_float(w[4] >> 16) * x.scale[1];
    return fmaf(sa, fmaf(-8.f, x.sum[0], (float)da), sb * fmaf(-8.f, x.sum[1], (float)db));
}

// d * (sc0 xs0 dot0 + sc1 xs1 dot1) - dmin * (m0 xs0 sum0 + m1 xs1 sum1) for the two sub-blocks of a
// pair (TransformerComputeKernelsQ4_K.java:651-667)
__device__ __forceinline__ float slice_dot_packed_q4_k(const uint4 &h, const uint4 &q0, const uint4 &q1,
                                                       int pair, const PackedX &x) {
    const uint32_t w[8] = {q0.x, q0.y, q0.z, q0.w, q1.x, q1.y, q1.z, q1.w};
    int d0 = 0, d1 = 0;
#pragma unroll
    for (int i = 0; i < 8; i++) {
        d0 = dot4(w[i] & 0x0F0F0F0Fu, x.q[i], d0);
        d1 = dot4((w[i] >> 4) & 0x0F0F0F0Fu, x.q[8 + i], d1);
    }
    int sc0, mn0, sc1, mn1;
    jl_q4k_scale_min(h.y, h.z, h.w, 2 * pair, sc0, mn0);
    jl_q4k_scale_min(h.y, h.z, h.w, 2 * pair + 1, sc1, mn1);
    const float d = jl_half_bits_to_float(h.x), dmin = jl_half_bits_to_float(h.x >> 16);
    const float scaled = fmaf((float)sc0 * x.scale[0], (float)d0, ((float)sc1 * x.scale[1]) * (float)d1);
    const float mins = fmaf((float)mn0 * x.scale[0], x.sum[0], ((float)mn1 * x.scale[1]) * x.sum[1]);
    return fmaf(d, scaled, -dmin * mins);
}

// ---- LDS access by hand ----------------------------------------------------------------------
//
// The tile stages are filled by LDS-DMA loads (global_load_lds_*), which the compiler tracks only
// coarsely: any LDS read it can see makes it wait for every outstanding vector-memory operation,
// which would drain the prefetch pipeline each tile.  All LDS traffic of the kernel therefore goes
// through inline assembly with explicit waits, and the workgroup barrier is the bare instruction.

typedef __attribute__((address_space(1))) const void gvoid;
typedef __attribute__((address_space(3))) void lvoid;

// s_waitcnt vmcnt(N) only (gfx9 encoding: vmcnt in bits 3:0 and 15:14, expcnt 6:4, lgkmcnt 11:8).
#define JL_WAIT_VM(N) \
    __builtin_amdgcn_s_waitcnt(((N)&0xF) | (((N) >> 4) << 14) | (0x7 << 4) | (0xF << 8))

// Waits until at most `tiles` tiles' worth of loads (PER_TILE each) are outstanding; every case is
// an immediate, as the instruction requires.
template <int PER_TILE>
__device__ __forceinline__ void wait_vm_tiles(int tiles) {
    switch (tiles) {
        case 0: JL_WAIT_VM(0); break;
        case 1: JL_WAIT_VM(PER_TILE); break;
        case 2: JL_WAIT_VM(2 * PER_TILE); break;
        case 3: JL_WAIT_VM(3 * PER_TILE); break;
        case 4: JL_WAIT_VM(4 * PER_TILE); break;
        case 5: JL_WAIT_VM(5 * PER_TILE); break;
        case 6: JL_WAIT_VM(6 * PER_TILE); break;
        default: JL_WAIT_VM(7 * PER_TILE); break;
    }
}

// two consecutive dwords from a four-byte aligned address
__device__ __forceinline__ uint2 lds_read_b64(uint32_t addr) {
    uint2 v;
    asm volatile("ds_read2_b32 %0, %1 offset0:0 offset1:1\n\ts_waitcnt lgkmcnt(0)" : "=&v"(v) : "v"(addr) : "memory");
    return v;
}

__device__ __forceinline__ uint32_t lds_read_b32(uint32_t addr) {
    uint32_t v;
    asm volatile("ds_read_b32 %0, %1\n\ts_waitcnt lgkmcnt(0)" : "=&v"(v) : "v"(addr) : "memory");
    return v;
}

__device__ __forceinline__ void lds_write_b32(uint32_t addr, uint32_t v) {
    asm volatile("ds_write_b32 %0, %1\n\ts_waitcnt lgkmcnt(0)" : : "v"(addr), "v"(v) : "memory");
}

typedef float floatx4 __attribute__((ext_vector_type(4)));
__device__ __forceinline__ void lds_write_x4(uint32_t addr, floatx4 v) {
    asm volatile("ds_write_b128 %0, %1\n\ts_waitcnt lgkmcnt(0)" : : "v"(addr), "v"(v) : "memory");
}

__device__ __forceinline__ void lds_read_x4(uint32_t addr, uint32_t (&w)[4]) {
    asm volatile("ds_read_b128 %0, %1\n\ts_waitcnt lgkmcnt(0)"
                 : "=&v"(*(uint4 *)w) : "v"(addr) : "memory");
}

// 16 activations' worth of registers (four 128-bit reads) with one wait
__device__ __forceinline__ void lds_read_16f(uint32_t addr, float *x) {
    float4 a, b, c, d;
    asm volatile(
        "ds_read_b128 %0, %4\n\tds_read_b128 %1, %4 offset:16\n\t"
        "ds_read_b128 %2, %4 offset:32\n\tds_read_b128 %3, %4 offset:48\n\ts_waitcnt lgkmcnt(0)"
        : "=&v"(a), "=&v"(b), "=&v"(c), "=&v"(d) : "v"(addr) : "memory");
    x[0] = a.x; x[1] = a.y; x[2] = a.z; x[3] = a.w;
    x[4] = b.x; x[5] = b.y; x[6] = b.z; x[7] = b.w;
    x[8] = c.x; x[9] = c.y; x[10] = c.z; x[11] = c.w;
    x[12] = d.x; x[13] = d.y; x[14] = d.z; x[15] = d.w;
}

// 17 consecutive dwords (one Q8_0 block pair): eight two-dword reads and one single
__device__ __forceinline__ void lds_read_17(uint32_t addr, uint32_t (&w)[17]) {
    uint2 p0, p1, p2, p3, p4, p5, p6, p7;
    uint32_t last;
    asm volatile(
        "ds_read2_b32 %0, %9 offset0:0 offset1:1\n\tds_read2_b32 %1, %9 offset0:2 offset1:3\n\t"
        "ds_read2_b32 %2, %9 offset0:4 offset1:5\n\tds_read2_b32 %3, %9 offset0:6 offset1:7\n\t"
        "ds_read2_b32 %4, %9 offset0:8 offset1:9\n\tds_read2_b32 %5, %9 offset0:10 offset1:11\n\t"
        "ds_read2_b32 %6, %9 offset0:12 offset1:13\n\tds_read2_b32 %7, %9 offset0:14 offset1:15\n\t"
        "ds_read_b32 %8, %9 offset:64\n\ts_waitcnt lgkmcnt(0)"
        : "=&v"(p0), "=&v"(p1), "=&v"(p2), "=&v"(p3), "=&v"(p4), "=&v"(p5), "=&v"(p6), "=&v"(p7),
          "=&v"(last)
        : "v"(addr) : "memory");
    w[0] = p0.x; w[1] = p0.y; w[2] = p1.x; w[3] = p1.y; w[4] = p2.x; w[5] = p2.y; w[6] = p3.x;
    w[7] = p3.y; w[8] = p4.x; w[9] = p4.y; w[10] = p5.x; w[11] = p5.y; w[12] = p6.x; w[13] = p6.y;
    w[14] = p7.x; w[15] = p7.y; w[16] = last;
}

// 9 consecutive dwords (one Q4_0 block pair)
__device__ __forceinline__ void lds_read_9(uint32_t addr, uint32_t (&w)[9]) {
    uint2 p0, p1, p2, p3;
    uint32_t last;
    asm volatile(
        "ds_read2_b32 %0, %5 offset0:0 offset1:1\n\tds_read2_b32 %1, %5 offset0:2 offset1:3\n\t"
        "ds_read2_b32 %2, %5 offset0:4 offset1:5\n\tds_read2_b32 %3, %5 offset0:6 offset1:7\n\t"
        "ds_read_b32 %4, %5 offset:32\n\ts_waitcnt lgkmcnt(0)"
        : "=&v"(p0), "=&v"(p1), "=&v"(p2), "=&v"(p3), "=&v"(last)
        : "v"(addr) : "memory");
    w[0] = p0.x; w[1] = p0.y; w[2] = p1.x; w[3] = p1.y; w[4] = p2.x; w[5] = p2.y; w[6] = p3.x;
    w[7] = p3.y; w[8] = last;
}

// a Q4_K super-block header (16 B) and the 32 nibble bytes of one pair
__device__ __forceinline__ void lds_read_q4k(uint32_t hdr, uint32_t qs, uint4 &h, uint4 &q0, uint4 &q1) {
    asm volatile(
        "ds_read_b128 %0, %3\n\tds_read_b128 %1, %4\n\tds_read_b128 %2, %4 offset:16\n\t"
        "s_waitcnt lgkmcnt(0)"
        : "=&v"(h), "=&v"(q0), "=&v"(q1) : "v"(hdr), "v"(qs) : "memory");
}

template <int TYPE>
__device__ __forceinline__ float slice_dot_lds(uint32_t stage, int r, int s, int row_bytes,
                                               const float (&x)[64], const float (&sx)[4]) {
    const uint32_t row = stage + (uint32_t)(r * row_bytes);
    if constexpr (TYPE == JL_IQ4_XS) {
        // the 8-byte header and the 32 nibble bytes of quarter s & 3 (super-blocks are 136 bytes
        // apart: everything is 8-byte aligned)
        const uint32_t sb = row + (s >> 2) * 136;
        uint2 hdr, a, b, c, e;
        asm volatile(
            "ds_read_b64 %0, %5\n\tds_read_b64 %1, %6\n\tds_read_b64 %2, %6 offset:8\n\t"
            "ds_read_b64 %3, %6 offset:16\n\tds_read_b64 %4, %6 offset:24\n\ts_waitcnt lgkmcnt(0)"
            : "=&v"(hdr), "=&v"(a), "=&v"(b), "=&v"(c), "=&v"(e) : "v"(sb), "v"(sb + 8 + (s & 3) * 32) : "memory");
        const uint32_t qs[8] = {a.x, a.y, b.x, b.y, c.x, c.y, e.x, e.y};
        return slice_dot_iq4_xs(hdr, qs, s & 3, x, sx);
    } else if constexpr (TYPE == JL_Q4_1) {
        // ten dwords, four-byte aligned (blocks are 20 bytes)
        uint32_t w9[9], w[10];
        lds_read_9(row + s * 40, w9);
        w[9] = lds_read_b32(row + s * 40 + 36);
#pragma unroll
        for (int i = 0; i < 9; i++) w[i] = w9[i];
        return slice_dot_q4_1(w, x, sx);
    } else if constexpr (TYPE == JL_Q5_0) {
        // eleven dwords from a four-byte aligned start (a pair of 22-byte blocks is 44 bytes); block
        // A's fields sit two bytes off the dwords: d | qh lo, qh hi | qs .., block B's on them
        uint32_t w9[9], w[11];
        lds_read_9(row + s * 44, w9);
        const uint2 t = lds_read_b64(row + s * 44 + 36);
#pragma unroll
        for (int i = 0; i < 9; i++) w[i] = w9[i];
        w[9] = t.x;
        w[10] = t.y;
        const uint32_t qh[2] = {__builtin_amdgcn_alignbit(w[1], w[0], 16), w[6]};
        uint32_t qs[8];
#pragma unroll
        for (int j = 0; j < 4; j++) {
            qs[j] = __builtin_amdgcn_alignbit(w[2 + j], w[1 + j], 16);
            qs[4 + j] = w[7 + j];
        }
        return slice_dot_q5_0(w[0], w[5] >> 16, qh, qs, x, sx);
    } else if constexpr (TYPE == JL_Q5_K) {
        // header, the 32 fifth-bit bytes, the 32 nibble bytes of pair s & 3 (super-blocks are 176
        // bytes apart: everything is 16-byte aligned)
        const uint32_t sb = row + (s >> 2) * 176;
        uint4 h, g0, g1, q0, q1;
        asm volatile(
            "ds_read_b128 %0, %5\n\tds_read_b128 %1, %5 offset:16\n\tds_read_b128 %2, %5 offset:32\n\t"
            "ds_read_b128 %3, %6\n\tds_read_b128 %4, %6 offset:16\n\ts_waitcnt lgkmcnt(0)"
            : "=&v"(h), "=&v"(g0), "=&v"(g1), "=&v"(q0), "=&v"(q1) : "v"(sb), "v"(sb + 48 + (s & 3) * 32) : "memory");
        const uint32_t qs[8] = {q0.x, q0.y, q0.z, q0.w, q1.x, q1.y, q1.z, q1.w};
        const uint32_t qh[8] = {g0.x, g0.y, g0.z, g0.w, g1.x, g1.y, g1.z, g1.w};
        return slice_dot_q5_k(h, qs, qh, s & 3, x, sx);
    } else if constexpr (TYPE == JL_Q6_K) {
        // Super-blocks are 210 bytes apart, so every other one starts two bytes off a dword.  The
        // LDS serves such reads, but at a fraction of its rate (measured: 40 % of the kernel's
        // time): the quarter is read as aligned dwords from two bytes before where that is needed
        // and each dword put together from its two neighbours with a funnel shift of 0 or 16 bits.
        const uint32_t sb = row + (s >> 2) * 210;
        const int h = (s >> 1) & 1;
        const uint32_t off = sb & 2u, shift = off * 8;
        uint32_t wl[17], wh[9], ql[16], qh[8];
        lds_read_17(sb - off + 64 * h, wl);
        lds_read_9(sb - off + 128 + 32 * h, wh);
        uint2 sc2;
        uint32_t d;
        asm volatile("ds_read2_b32 %0, %2 offset0:0 offset1:1\n\tds_read_u16 %1, %3\n\ts_waitcnt lgkmcnt(0)"
                     : "=&v"(sc2), "=&v"(d) : "v"(sb - off + 192 + 4 * (s & 3)), "v"(sb + 208) : "memory");
#pragma unroll
        for (int i = 0; i < 16; i++) ql[i] = __builtin_amdgcn_alignbit(wl[i + 1], wl[i], shift);
#pragma unroll
        for (int i = 0; i < 8; i++) qh[i] = __builtin_amdgcn_alignbit(wh[i + 1], wh[i], shift);
        const uint32_t scales = __builtin_amdgcn_alignbit(sc2.y, sc2.x, shift);
        return slice_dot_q6_k(ql, qh, scales, d, s & 1, x, sx);
    } else if constexpr (TYPE == JL_Q8_0) {
        uint32_t w[17];
        lds_read_17(row + s * 68, w);
        return slice_dot_q8_0(w, x);
    } else if constexpr (TYPE == JL_Q4_0) {
        uint32_t w[9];
        lds_read_9(row + s * 36, w);
        return slice_dot_q4_0(w, x, sx);
    } else {
        uint4 h, q0, q1;
        uint32_t sb = row + (s >> 2) * 144;
        lds_read_q4k(sb, sb + 16 + (s & 3) * 32, h, q0, q1);
        return slice_dot_q4_k(h, q0, q1, s & 3, x, sx);
    }
}

template <int TYPE>
__device__ __forceinline__ float slice_dot_lds_packed(uint32_t stage, int r, int s, int row_bytes, const PackedX &x) {
    const uint32_t row = stage + (uint32_t)(r * row_bytes);
    if constexpr (TYPE == JL_Q8_0) {
        uint32_t w[17];
        lds_read_17(row + s * 68, w);
        return slice_dot_packed_q8_0(w, x);
    } else if constexpr (TYPE == JL_Q4_0) {
        uint32_t w[9];
        lds_read_9(row + s * 36, w);
        return slice_dot_packed_q4_0(w, x);
    } else {
        uint4 h, q0, q1;
        uint32_t sb = row + (s >> 2) * 144;
        lds_read_q4k(sb, sb + 16 + (s & 3) * 32, h, q0, q1);
        return slice_dot_packed_q4_k(h, q0, q1, s & 3, x);
    }
}

// Cache policy bit of the weight stream's LDS-DMA loads: the fused gate/up form, which reads two
// weights tile by tile in turn, marks its loads non-temporal (bit 1 of the instruction's cache
// policy).  Measured on the 2 x [8192 x 2048] Q8_0 launch: 8.15 -> 7.93 us; the single-weight launches
// are 3-6 % slower with the same mark and keep the default policy.  (A plain constant: as a variable
// template in this unnamed namespace it left the host side without the kernels' launch stubs.)
constexpr int kStreamNonTemporal = 2;

// LDS map: [0, kPartialBytes) row partial sums, two parities; then the stage ring.  The activation
// vector is staged in the ring's last stage (or, when it is larger than a stage, in a region of
// its own after the ring) until every thread holds its 64 activations in registers.
constexpr int kPartialBytes = 2048;  // 2 parities x 256 floats
// Depth of the LDS tile ring: one tile computed, one in flight.  Measured on every benchmark shape,
// a deeper ring at the lower occupancy its LDS footprint forces is slower (and no faster where it
// costs no occupancy: the 9 KB tiles of the 4-bit types at 3 and 4 stages).
constexpr int kStages = 2;
constexpr int kWideThreads = 1024;   // workgroup of the plain kernel for rows of more than 128 slices

// v + (the value two quad neighbours hold): DPP quad permutes, VALU speed, no LDS round trip
__device__ __forceinline__ float quad_xor1(float v) {
    return __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(v), 0xB1, 0xF, 0xF, true));
}
__device__ __forceinline__ float quad_xor2(float v) {
    return __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(v), 0x4E, 0xF, 0xF, true));
}

// RMS: the activations are RMS-normalised on their way in (a variant of its own, so that the plain
// kernel's registers and schedule are not touched by it).
// Hands a loaded argument back as a plain scalar value.  Without it the compiler merges "this
// local or that argument-array element" into one pointer and loads through it with a flat load,
// whose wait drains the tile ring every tile.
__device__ __forceinline__ uint32_t uniform_value(uint32_t v) {
    asm volatile("" : "+s"(v));
    return v;
}
__device__ __forceinline__ uintptr_t uniform_value(uintptr_t v) {
    asm volatile("" : "+s"(v));
    return v;
}


// SPT != 0 is the kernel for the usual launch, with its geometry known to the compiler: rows of
// exactly SPT slices (a power of two), THREADS / SPT rows per tile and, in every segment, a row
// count that is a multiple of that, so every thread has a slice, every tile is whole and every
// output row exists.  Sizes, offsets, the lane folds and the choice between the two ways of
// finishing a row are then constants and most of the loop's branches and scalar bookkeeping (226
// scalar instructions per tile and wave in the general form, as many as the vector ones) are gone.
// (SEGS: the fixed-geometry form of the fused q|k|v, up to three weights side by side.)
// (PART: rows of fewer than SPT slices -- 11 008, 12 288, 14 336 columns under SPT = 256 -- whose
// lanes past the row's end idle; everything but the row length is still a constant.)
// (ARGMAX: a plain projection whose rows lie inside a wave also keeps, per workgroup, the largest
// value it stored and that value's row -- greedy sampling then folds a thousand cells instead of
// reading the logits back.)
// (HALVES: rows of more than 256 slices, up to 512 -- 16 448 to 32 768 columns, the down projections of
// the largest models.  A row of 2 m columns is, byte for byte, two consecutive rows of m columns, so
// the launch describes the weight as [2 d x m]: even rows meet the first half of the activation
// vector, odd rows the second.  A tile holds four such half rows, so a thread always serves the same
// half and keeps its 64 activations in registers as ever; they come straight from global memory, as
// the vector is longer than a ring stage.  The thread that finishes a row adds its two halves'
// partial sums.)
template <int TYPE, bool DUAL, bool RMS, bool PACKED = false, int THREADS = 256, int SPT = 0, bool SEGS = false,
          bool PART = false, bool ARGMAX = false, bool HALVES = false>
__global__ void __launch_bounds__(THREADS) jl_gemv_tiles(const uint8_t *w_first, const uint8_t *w_up_first, const float *x_first, int tiles_first,
              int rows_first, int grid_first, int S_first, int row_bytes_first, int shape_first,
              const float *rms_w_first, GemvParams p) {
    // The leading arguments repeat what the kernel needs before its first tile's loads can go out
    // (first weight, up weight, the activation vector, tile count, first weight's rows, grid width,
    // slices and bytes of a row, padded slices | rows per tile << 10 | weights << 20 for the general
    // form, the RMS weights):
    // the build preloads them into scalar registers at dispatch (-amdgpu-kernarg-preload-count),
    // where a read of the argument buffer is a round trip to memory at the head of every launch.
    // (Preloading the q|k|v form's other two weights and first tiles as well changed nothing.)
    static_assert(!(RMS && PACKED), "the packed activation is normalised before it is quantised");
    constexpr bool LEAN = SPT != 0;
    constexpr bool FULL = LEAN && !PART;   // every lane has a slice, every load slot is real data
    static_assert(!PART || LEAN, "rows shorter than SPT slices: a fixed tile shape");
    static_assert(!LEAN || !PACKED, "the packed form has no fixed-geometry instances");
    static_assert(!ARGMAX || (FULL && !DUAL && !SEGS && SPT <= 64), "the argmax form: whole in-wave rows of one weight");
    static_assert(!HALVES || (PART && !DUAL && !RMS && !PACKED && !SEGS && !ARGMAX && THREADS == 1024 && SPT == 256),
                  "rows in two halves: the plain 1024-thread form");
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    constexpr int X4 = Traits<TYPE>::kX4;        // 16-byte loads per thread and tile
    constexpr int L = X4 + Traits<TYPE>::kTail;   // plus (three main types) one 4-byte load
    constexpr int SLICE = X4 * 16 + 4 * Traits<TYPE>::kTail;   // bytes of a tile one thread brings in
    constexpr bool kExactDma = is_main_type(TYPE);   // a thread's loads are exactly its slice

    const int tid = threadIdx.x;
    const int nthreads = LEAN ? THREADS : (int)blockDim.x;
    // geometry: constants in the fixed-geometry form, launch arguments otherwise
    const int Sp = LEAN ? SPT : (shape_first & 0x3FF), S = FULL ? SPT : S_first;
    const int R = LEAN ? THREADS / (LEAN ? SPT : 1) : ((shape_first >> 10) & 0x3FF);
    const int row_bytes = FULL ? row_bytes_of<TYPE>(SPT) : row_bytes_first;
    const int wave = __builtin_amdgcn_readfirstlane(tid / JL_WAVE);   // uniform: LDS-DMA bases stay scalar
    const int lane = tid & (JL_WAVE - 1);
    const int r = tid / Sp;           // row of the tile this thread works on
    const int s = tid - r * Sp;       // its 64-column slice
    const bool active = FULL || ((s < S) && (LEAN || r < R));
    const int half_rows = DUAL ? R / 2 : R;       // output rows per tile
    const int half_bytes = half_rows * row_bytes;   // bytes of a tile that come from one weight
    const int nseg = (LEAN && !SEGS) ? 1 : ((shape_first >> 20) & 0xF);
    const int total_tiles = tiles_first;
    const int stage_bytes = nthreads * SLICE;
    // every thread of the workgroup owns a slice and every load slot is real data
    const bool exact = kExactDma && (FULL || (!PART && (S == Sp) && (R * Sp == nthreads)));

    const uint32_t lds0 = (uint32_t)(uintptr_t)(lvoid *)lds;
    const uint32_t ring0 = lds0 + kPartialBytes;
    uint8_t *ring = lds + kPartialBytes;

    // Per-thread byte offsets of its L load slots inside a tile; for a gate/up tile the slots past
    // half_bytes read the up weight.
    int slot_off[L];
    bool slot_up[L];
#pragma unroll
    for (int k = 0; k < L; k++) {
        int off = k < X4 ? (k * nthreads + tid) * 16 : X4 * nthreads * 16 + tid * 4;
        slot_up[k] = DUAL && off >= half_bytes;
        slot_off[k] = slot_up[k] ? off - half_bytes : off;
    }

    // Brings tile `tile` into stage `st`.  Every thread issues exactly L loads, whatever the tile:
    // lanes that have nothing to fetch re-read the segment's first bytes into their own slot, so
    // each wave's outstanding-load count is a compile-time constant per tile.
    // (a launch with one segment -- every one but the fused q|k|v -- never indexes the argument
    // arrays with a run-time segment: that is a scalar memory load, and a wait, per tile)
    const uint8_t *const w0 = w_first;
    const int rows0 = rows_first;
    float *const out0 = p.out[0];
    auto segment_of = [&](int tile) {
        int seg = 0;
#pragma unroll
        for (int i = 1; i < kMaxSeg; i++)
            if (i < nseg && tile >= p.seg_tile_begin[i]) seg = i;
        return seg;
    };
    // The fixed-geometry form keeps every segment's bases in scalar registers (the argument arrays
    // read with constant indices, once) and picks by comparing the tile with the segments' first
    // tiles: no memory access per tile at all.
    const uint8_t *seg_w[kMaxSeg] = {};
    float *seg_out[kMaxSeg] = {};
    int seg_begin[kMaxSeg] = {};
    if constexpr (LEAN && SEGS) {
#pragma unroll
        for (int i = 0; i < kMaxSeg; i++) {
            seg_w[i] = p.w[i];
            seg_out[i] = p.out[i];
            seg_begin[i] = p.seg_tile_begin[i];
        }
    }
    auto issue = [&](int tile, int st) {
        const uint8_t *wseg = w0;
        int seg_rows = rows0, local = tile;
        if (nseg > 1) {
            if constexpr (LEAN) {
#pragma unroll
                for (int i = 1; i < kMaxSeg; i++)
                    if (i < nseg && tile >= seg_begin[i]) {
                        wseg = seg_w[i];
                        local = tile - seg_begin[i];
                    }
            } else {
                const int seg = segment_of(tile);
                wseg = (const uint8_t *)uniform_value((uintptr_t)p.w[seg]);
                seg_rows = (int)uniform_value((uint32_t)p.seg_rows[seg]);
                local = tile - (int)uniform_value((uint32_t)p.seg_tile_begin[seg]);
            }
        }
        const int64_t offset = (int64_t)local * half_bytes;
        const int64_t remain = (int64_t)seg_rows * row_bytes - offset;
        // (the fixed-geometry form is launched over whole tiles only, and tracks no segment's rows)
        const int bytes = LEAN || remain >= half_bytes ? half_bytes : (int)remain;
        const uint8_t *base = wseg + offset;
        const uint8_t *base_up = DUAL ? w_up_first + offset : base;
        uint8_t *dst = ring + st * stage_bytes;
        const bool whole = exact && (FULL || bytes == half_bytes);  // uniform
        if (whole) {
            // the usual case (uniform): every slot is inside the tile, nothing to redirect
#pragma unroll
            for (int k = 0; k < L; k++) {
                const int wave_off = k < X4 ? (k * nthreads + wave * JL_WAVE) * 16
                                            : X4 * nthreads * 16 + wave * JL_WAVE * 4;
                const uint8_t *src = (DUAL && slot_up[k] ? base_up : base) + slot_off[k];
                if (k < X4)
                    __builtin_amdgcn_global_load_lds((gvoid *)src, (lvoid *)(dst + wave_off), 16, 0, DUAL ? kStreamNonTemporal : 0);
                else
                    __builtin_amdgcn_global_load_lds((gvoid *)src, (lvoid *)(dst + wave_off), 4, 0, DUAL ? kStreamNonTemporal : 0);
            }
        } else {
#pragma unroll
            for (int k = 0; k < L; k++) {
                const int width = k < X4 ? 16 : 4;
                const int wave_off = k < X4 ? (k * nthreads + wave * JL_WAVE) * 16
                                            : X4 * nthreads * 16 + wave * JL_WAVE * 4;
                const uint8_t *src = (DUAL && slot_up[k] ? base_up : base) + slot_off[k];
                if (slot_off[k] + width > bytes) src = wseg;
                if (k < X4)
                    __builtin_amdgcn_global_load_lds((gvoid *)src, (lvoid *)(dst + wave_off), 16, 0, 0);
                else
                    __builtin_amdgcn_global_load_lds((gvoid *)src, (lvoid *)(dst + wave_off), 4, 0, 0);
            }
        }
    };
    // my tiles: blockIdx.x, blockIdx.x + grid, ...
    const int grid = grid_first;
    const int first = blockIdx.x;
    const int mine = first < total_tiles ? (total_tiles - first + grid - 1) / grid : 0;

    // Segmented sum over aligned groups of `width` lanes (a power of two): row-local DPP moves up
    // to 16 lanes, cross-row permutes beyond.
    auto group_sum = [&](float v, int width) {
        if (width >= 2) v += quad_xor1(v);
        if (width >= 4) v += quad_xor2(v);
        if (width >= 8)
            v += __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(v), 0x141, 0xF, 0xF, true));
        if (width >= 16)
            v += __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(v), 0x140, 0xF, 0xF, true));
        if (width >= 32) v += __shfl_xor(v, 16, JL_WAVE);
        if (width >= 64) v += __shfl_xor(v, 32, JL_WAVE);
        return v;
    };

    constexpr bool rms = RMS;

    // Activations first (oldest loads), then the first stages - 1 tiles.  In LDS a thread's 64
    // activations take 17 sixteen-byte slots, the last one padding: slices then start 272 bytes
    // apart and the 128-bit reads below spread over all banks (256 bytes apart they would all
    // land on the same four).  Slot q holds floats 64 * (q / 17) + 4 * (q % 17) ... + 3.
    const int x_slots = S * 17;
    const int x_bytes = (x_slots + nthreads - 1) / nthreads * nthreads * 16;
    const bool x_in_ring = x_bytes <= stage_bytes;  // else a region of its own after the ring
    uint8_t *xs = x_in_ring ? ring + (kStages - 1) * stage_bytes : ring + kStages * stage_bytes;
    const uint32_t xs0 = x_in_ring ? ring0 + (kStages - 1) * stage_bytes : ring0 + kStages * stage_bytes;
    int issued = 0;
    if constexpr (!rms && !PACKED && !HALVES) {
        for (int base = 0; base < x_bytes; base += nthreads * 16) {
            const int q = base / 16 + tid;
            const int sl = q / 17, k = q - sl * 17;
            const int off = (sl < S && k < 16) ? (sl * 64 + k * 4) * 4 : 0;
            // (the side types' vector region, where it is one of its own, ends with the vector's last
            // slot -- their 1024-thread form fits the LDS only so -- and nothing is written past it)
            if (kExactDma || x_in_ring || q < x_slots)
                __builtin_amdgcn_global_load_lds((gvoid *)((const uint8_t *)x_first + off),
                                                 (lvoid *)(xs + base + wave * JL_WAVE * 16), 16, 0, 0);
        }
    }
    // RMS normalisation folded into the activation load.  CpuOperations.rmsnorm
    // (J/inference/op/CpuOperations.java:60-72): out = w * (ss * x) with
    // ss = (float)(1 / sqrt(sum x^2 / n + eps)); the reference's fused kernels fold the same
    // product into their activation reads (TransformerComputeKernelsLayered.java:2168-2171).
    // The workgroup reads x and the weights with coalesced 16-byte loads and leaves the
    // product in the LDS region the plain path fills with x, so everything after is shared
    // and the LDS footprint (workgroups per compute unit) is that of the plain path.
    const int nvec = rms ? p.n / 4 : 0;
    const float4 *xv = (const float4 *)x_first, *wv = (const float4 *)rms_w_first;
    // rows of up to kHold x 4 x nthreads columns are read once and held in registers from the
    // sum of squares to the product; longer ones are read again for the product (the
    // fixed-geometry form's rows always fit: SPT slices of 64 columns)
    constexpr int kHold = LEAN ? (SPT * 16 / THREADS > 1 ? SPT * 16 / THREADS : 1) : 4;
    const bool held = LEAN || nvec <= nthreads * kHold;
    float4 v[kHold], w[kHold];
    auto load = [&](int base) {
#pragma unroll
        for (int j = 0; j < kHold; j++) {
            const int i = base + j * nthreads + tid;
            v[j] = i < nvec ? xv[i] : float4{0.f, 0.f, 0.f, 0.f};
            w[j] = i < nvec ? wv[i] : float4{0.f, 0.f, 0.f, 0.f};
        }
    };
    // (these loads go out before the first tile's: a wait for them then leaves the tile in flight
    // while the sum of squares and the products are computed, instead of waiting for it as well)
    if constexpr (rms) {
        if (held) load(0);
    }
    for (; issued < kStages - 1 && issued < mine; issued++) issue(first + issued * grid, issued);
    if constexpr (rms) {
        float scale;
        if (p.rms_scale) {
            scale = *p.rms_scale;
        } else {
            float ss = 0.f;
            if (held) {
#pragma unroll
                for (int j = 0; j < kHold; j++) {
                    ss = fmaf(v[j].x, v[j].x, ss);
                    ss = fmaf(v[j].y, v[j].y, ss);
                    ss = fmaf(v[j].z, v[j].z, ss);
                    ss = fmaf(v[j].w, v[j].w, ss);
                }
            } else {
                for (int i = tid; i < nvec; i += nthreads) {
                    const float4 u = xv[i];
                    ss = fmaf(u.x, u.x, ss);
                    ss = fmaf(u.y, u.y, ss);
                    ss = fmaf(u.z, u.z, ss);
                    ss = fmaf(u.w, u.w, ss);
                }
            }
            // wave sums meet in the last words of the partial-sum region, which nothing else
            // touches before the first tile is finished
            ss = group_sum(ss, JL_WAVE);
            const uint32_t cell = lds0 + kPartialBytes - 64;
            if (lane == 0) lds_write_b32(cell + wave * 4, __float_as_uint(ss));
            __builtin_amdgcn_s_barrier();
            ss = 0.f;
            for (int i = 0; i < nthreads / JL_WAVE; i++) ss += __uint_as_float(lds_read_b32(cell + i * 4));
            scale = (float)(1.0 / sqrt((double)(ss / (float)p.n + p.rms_eps)));
        }
        for (int base = 0; base < nvec; base += nthreads * kHold) {
            if (!held) load(base);
#pragma unroll
            for (int j = 0; j < kHold; j++) {
                const int i = base + j * nthreads + tid;
                if (i < nvec) {
                    const floatx4 o = {w[j].x * (scale * v[j].x), w[j].y * (scale * v[j].y),
                                       w[j].z * (scale * v[j].z), w[j].w * (scale * v[j].w)};
                    lds_write_x4(xs0 + ((i >> 4) * 17 + (i & 15)) * 16, o);
                }
            }
        }
    }
    wait_vm_tiles<L>(issued);
    __builtin_amdgcn_s_barrier();

    float x[64];
    float sx[4] = {0.f, 0.f, 0.f, 0.f};   // sums of the slice's activations by 32 (4-bit types) or 16 (Q6_K)
    PackedX px;
    if constexpr (PACKED) {
        // the slice's 64 bytes, two scales and two sums straight from global memory (a few KB that
        // every workgroup reads: they stay in the cache)
        uint32_t raw[16];
#pragma unroll
        for (int k = 0; k < 16; k++) raw[k] = 0;
        px.scale[0] = px.scale[1] = px.sum[0] = px.sum[1] = 0.f;
        if (active) {
            const uint4 *src = (const uint4 *)(p.xq + s * 64);
#pragma unroll
            for (int k = 0; k < 4; k++) {
                const uint4 v = src[k];
                raw[4 * k] = v.x; raw[4 * k + 1] = v.y; raw[4 * k + 2] = v.z; raw[4 * k + 3] = v.w;
            }
            const float2 sc = *(const float2 *)(p.xq_scales + 2 * s);
            const int2 sm = *(const int2 *)(p.xq_sums + 2 * s);
            px.scale[0] = sc.x; px.scale[1] = sc.y;
            px.sum[0] = (float)sm.x; px.sum[1] = (float)sm.y;
        }
        pack_x<TYPE>(raw, px);
    } else {
        // (threads with no slice never use theirs: the dot product below is skipped for them)
        if constexpr (HALVES) {
            if (active) {
                const float4 *src = (const float4 *)(x_first + ((r & 1) * S + s) * 64);
#pragma unroll
                for (int k = 0; k < 16; k++) {
                    const float4 v4 = src[k];
                    x[4 * k] = v4.x; x[4 * k + 1] = v4.y; x[4 * k + 2] = v4.z; x[4 * k + 3] = v4.w;
                }
            }
        } else if (active) {
#pragma unroll
            for (int k = 0; k < 4; k++) lds_read_16f(xs0 + s * 272 + k * 64, &x[k * 16]);
        }
        if constexpr (TYPE == JL_Q6_K) {
#pragma unroll
            for (int k = 0; k < 16; k++) {
                sx[0] += x[k];
                sx[1] += x[16 + k];
                sx[2] += x[32 + k];
                sx[3] += x[48 + k];
            }
        } else if constexpr (TYPE != JL_Q8_0) {   // Q4_0, Q4_K, Q5_K: by 32
#pragma unroll
            for (int k = 0; k < 32; k++) {
                sx[0] += x[k];
                sx[1] += x[32 + k];
            }
        }
    }

    // A row's Sp lane sums are folded over quads in registers, then one lane per quad leaves its
    // partial in LDS and the row's finishing thread adds the P = Sp / 4 partials one tile later.
    const int P = Sp >= 4 ? Sp / 4 : 1;
    constexpr uint32_t kParity = kPartialBytes / 2;

    // Finishes tile `t` from the partials of parity `par`.  The R * P partial slots are at most
    // 64 when P >= 1 quad per row, so wave 0 takes one slot per lane, folds each row's P lanes and
    // lets the row's first lane apply the epilogue; narrower rows (P == 1) take one thread each.
    auto finish = [&](int t, int par) {
        const int slots = half_rows * P;
        if (tid < slots) {
            const uint32_t pb = lds0 + par * kParity;
            float v0 = __uint_as_float(lds_read_b32(pb + tid * 4));
            float v1 = 0.f;
            if constexpr (DUAL) v1 = __uint_as_float(lds_read_b32(pb + (slots + tid) * 4));
            // (the row's other half lies P partials further on, or back)
            if constexpr (HALVES) v0 += __uint_as_float(lds_read_b32(pb + (tid ^ P) * 4));
            if (P > 1) {
                const int width = P < JL_WAVE ? P : JL_WAVE;
                v0 = group_sum(v0, width);
                if constexpr (DUAL) v1 = group_sum(v1, width);
            }
            const int j = tid / P;  // row of the tile
            int local = t, seg_rows = rows0;
            float *out = out0;
            if (nseg > 1) {
                if constexpr (LEAN) {
#pragma unroll
                    for (int i = 1; i < kMaxSeg; i++)
                        if (i < nseg && t >= seg_begin[i]) {
                            out = seg_out[i];
                            local = t - seg_begin[i];
                        }
                } else {
                    const int seg = segment_of(t);
                    local = t - (int)uniform_value((uint32_t)p.seg_tile_begin[seg]);
                    seg_rows = (int)uniform_value((uint32_t)p.seg_rows[seg]);
                    out = (float *)uniform_value((uintptr_t)p.out[seg]);
                }
            }
            const int row = local * half_rows + j;
            if (tid - j * P == 0 && (LEAN || row < seg_rows) && (!HALVES || (j & 1) == 0)) {
                float *o = out + (HALVES ? row >> 1 : row);
                if constexpr (DUAL) {
                    *o = jl_swiglu_value(v0, v1);
                } else {
                    // no read-modify-write through a load: a load's wait would drain the prefetch ring
                    if (p.epilogue == JL_RESIDUAL) unsafeAtomicAdd(o, v0);
                    else *o = v0;
                }
            }
        }
    };

    // Rows of at most 64 slices lie inside one wave: their lane sums are folded in registers and the
    // row's first lane applies the epilogue itself -- no partial sums in LDS, no finishing pass one
    // tile later, no barrier behind the last tile.  For gate/up the rows are dealt gate 0, up 0,
    // gate 1, up 1, ... so that both halves of an output sit in the same wave (rows of 64 slices
    // fill a wave each, so gate/up keeps the LDS hand-over there).
    const bool in_wave = Sp <= (DUAL ? 32 : 64);
    const int r_lds = (DUAL && in_wave) ? (r & 1) * half_rows + (r >> 1) : r;   // tile row this thread reads
    float best = -INFINITY;   // ARGMAX: the largest value this lane has stored, and its row
    int best_at = INT_MAX;
    for (int it = 0; it < mine; it++) {
        const int tile = first + it * grid;
        // with two stages nothing was issued after tile `it`: its loads are the youngest
        JL_WAIT_VM(0);
        __builtin_amdgcn_s_barrier();
        // the stage that tile it - 1 (or, the first time round, the activation vector) occupied
        // is free now: every wave is past its reads
        if (issued < mine) {
            issue(first + issued * grid, issued % kStages);
            issued++;
        }
        if (!in_wave && it > 0) finish(tile - grid, (it - 1) & 1);

        float v = 0.f;
        if (active) {
            if constexpr (PACKED) v = slice_dot_lds_packed<TYPE>(ring0 + (it % kStages) * stage_bytes, r_lds, s, row_bytes, px);
            else v = slice_dot_lds<TYPE>(ring0 + (it % kStages) * stage_bytes, r_lds, s, row_bytes, x, sx);
        }
        if (in_wave) {
            v = group_sum(v, Sp);
            float up = 0.f;
            if constexpr (DUAL) up = __shfl(v, lane + Sp, JL_WAVE);   // the up row sits Sp lanes on
            const int j = DUAL ? r >> 1 : r;   // output row of the tile
            if (s == 0 && (LEAN || r < R) && (!DUAL || (r & 1) == 0)) {
                int local = tile, seg_rows = rows0;
                float *out = out0;
                if (nseg > 1) {
                    if constexpr (LEAN) {
#pragma unroll
                        for (int i = 1; i < kMaxSeg; i++)
                            if (i < nseg && tile >= seg_begin[i]) {
                                out = seg_out[i];
                                local = tile - seg_begin[i];
                            }
                    } else {
                        const int seg = segment_of(tile);
                        local = tile - (int)uniform_value((uint32_t)p.seg_tile_begin[seg]);
                        seg_rows = (int)uniform_value((uint32_t)p.seg_rows[seg]);
                        out = (float *)uniform_value((uintptr_t)p.out[seg]);
                    }
                }
                const int row = local * half_rows + j;
                if (LEAN || row < seg_rows) {
                    float *o = out + row;
                    if constexpr (DUAL) {
                        *o = jl_swiglu_value(v, up);
                    } else {
                        // no read-modify-write through a load: a load's wait would drain the prefetch ring
                        if (p.epilogue == JL_RESIDUAL) unsafeAtomicAdd(o, v);
                        else *o = v;
                        if constexpr (ARGMAX) {
                            // a lane's rows ascend: the strict comparison keeps the first of equals
                            if (v > best) {
                                best = v;
                                best_at = row;
                            }
                        }
                    }
                }
            }
            continue;
        }
        if (Sp >= 2) v += quad_xor1(v);
        if (Sp >= 4) v += quad_xor2(v);
        if ((LEAN || r < R) && (Sp < 4 ? s == 0 : (s & 3) == 0)) {
            const int slot = r * P + (s >> 2);
            lds_write_b32(lds0 + (it & 1) * kParity + slot * 4, __float_as_uint(v));
        }
    }
    if (mine > 0 && !in_wave) {
        __builtin_amdgcn_s_barrier();
        finish(first + (mine - 1) * grid, (mine - 1) & 1);
    }
    if constexpr (ARGMAX) {
        // larger value wins, equal values: the lower row.  Lanes, then waves through the (unused,
        // rows being in-wave) partial-sum region, then one cell per workgroup.
        auto keep_better = [](float &v, int &i, float ov, int oi) {
            if (ov > v || (ov == v && oi < i)) {
                v = ov;
                i = oi;
            }
        };
#pragma unroll
        for (int o = JL_WAVE / 2; o > 0; o >>= 1) {
            const float ov = __shfl_xor(best, o, JL_WAVE);
            const int oi = __shfl_xor(best_at, o, JL_WAVE);
            keep_better(best, best_at, ov, oi);
        }
        if (lane == 0) {
            lds_write_b32(lds0 + wave * 8, __float_as_uint(best));
            lds_write_b32(lds0 + wave * 8 + 4, (uint32_t)best_at);
        }
        __builtin_amdgcn_s_barrier();
        if (tid == 0) {
            for (int i = 1; i < THREADS / JL_WAVE; i++)
                keep_better(best, best_at, __uint_as_float(lds_read_b32(lds0 + i * 8)), (int)lds_read_b32(lds0 + i * 8 + 4));
            p.best_value[blockIdx.x] = best;
            p.best_index[blockIdx.x] = best_at;
        }
    }
}

// Catch-all for shapes the tile kernel does not take (row length not a multiple of 64, rows wider
// than 16384 columns that the two-halves form does not take either, unaligned buffers): one wave per
// row, lanes stride over blocks, byte loads.
template <int TYPE>
__device__ float block_dot_generic(const uint8_t *blk, const float *x) {
    float acc = 0.f;
    if constexpr (TYPE == JL_Q8_0) {
        float d = jl_half_bits_to_float(blk[0] | (blk[1] << 8));
        for (int i = 0; i < 32; i++) acc = fmaf((float)(int)(int8_t)blk[2 + i], x[i], acc);
        return acc * d;
    } else if constexpr (TYPE == JL_Q4_0) {
        float d = jl_half_bits_to_float(blk[0] | (blk[1] << 8));
        for (int i = 0; i < 16; i++) {
            int b = blk[2 + i];
            acc = fmaf((float)((b & 0xF) - 8), x[i], acc);
            acc = fmaf((float)((b >> 4) - 8), x[16 + i], acc);
        }
        return acc * d;
    } else {
        const uint32_t *hdr = (const uint32_t *)blk;
        float d = jl_half_bits_to_float(hdr[0]);
        float dmin = jl_half_bits_to_float(hdr[0] >> 16);
        for (int j = 0; j < 8; j++) {
            int sc, mn;
            jl_q4k_scale_min(hdr[1], hdr[2], hdr[3], j, sc, mn);
            float qx = 0.f, sx = 0.f;
            const uint8_t *qs = blk + 16 + (j >> 1) * 32;
            for (int i = 0; i < 32; i++) {
                int q = (j & 1) ? (qs[i] >> 4) : (qs[i] & 0xF);
                qx = fmaf((float)q, x[j * 32 + i], qx);
                sx += x[j * 32 + i];
            }
            acc += (d * (float)sc) * qx - (dmin * (float)mn) * sx;
        }
        return acc;
    }
}

template <int TYPE>
__global__ void __launch_bounds__(256)
jl_gemv_generic(const uint8_t *__restrict__ w, const uint8_t *__restrict__ w_up,
                const float *__restrict__ x, float *__restrict__ out, int rows, int n, int epilogue) {
    constexpr int BE = TYPE == JL_Q4_K ? 256 : 32;
    constexpr int BB = TYPE == JL_Q4_K ? 144 : TYPE == JL_Q8_0 ? 34 : 18;
    int row = blockIdx.x * (blockDim.x / JL_WAVE) + threadIdx.x / JL_WAVE;
    int lane = threadIdx.x & (JL_WAVE - 1);
    if (row >= rows) return;
    int blocks = n / BE;
    const uint8_t *wr = w + (int64_t)row * blocks * BB;
    float v0 = 0.f, v1 = 0.f;
    for (int b = lane; b < blocks; b += JL_WAVE) {
        v0 += block_dot_generic<TYPE>(wr + (int64_t)b * BB, x + b * BE);
        if (w_up) v1 += block_dot_generic<TYPE>(w_up + ((int64_t)row * blocks + b) * BB, x + b * BE);
    }
    v0 = jl_group_sum<JL_WAVE>(v0);
    v1 = jl_group_sum<JL_WAVE>(v1);
    if (lane == 0) {
        if (epilogue == JL_SWIGLU) out[row] = jl_swiglu_value(v0, v1);
        else if (epilogue == JL_RESIDUAL) out[row] += v0;
        else out[row] = v0;
    }
}

// ---- host side ------------------------------------------------------------------------------

// LDS of a workgroup of `threads`: partial sums, the tile ring, and the staged activation vector
// where it is larger than a ring stage.
int tile_lds_bytes(int threads, int slice, int S, bool exact_vector_region = false) {
    const int stage_bytes = threads * slice;
    const int x_bytes = (S * 17 + threads - 1) / threads * threads * 16;  // 17 slots per slice
    const int x_extra = x_bytes <= stage_bytes ? 0 : exact_vector_region ? S * 17 * 16 : x_bytes;
    return kPartialBytes + kStages * stage_bytes + x_extra;
}

int next_pow2(int v) {
    int p = 1;
    while (p < v) p <<= 1;
    return p;
}

struct OccKey {
    const void *fn;
    int device, threads, lds;
    bool operator<(const OccKey &o) const {
        return std::tie(fn, device, threads, lds) < std::tie(o.fn, o.device, o.threads, o.lds);
    }
};

// Workgroups of `fn` that fit one compute unit; asked of the runtime once per configuration.
int blocks_per_cu(const void *fn, int device, int threads, int lds) {
    static std::mutex mu;
    static std::map<OccKey, int> cache;
    std::lock_guard<std::mutex> g(mu);
    OccKey key{fn, device, threads, lds};
    auto it = cache.find(key);
    if (it != cache.end()) return it->second;
    (void)hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
    int nb = 0;
    if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&nb, fn, threads, (size_t)lds) != hipSuccess ||
        nb < 1) {
        (void)hipGetLastError();
        nb = 1;
    }
    cache[key] = nb;
    return nb;
}

template <int TYPE, bool DUAL, bool RMS, bool PACKED = false, int THREADS = 256, int SPT = 0, bool SEGS = false,
          bool PART = false, bool ARGMAX = false, bool HALVES = false>
int launch_tiles_of(jl_context *ctx, const GemvParams &p, int threads, int lds, int *cells = nullptr) {
    auto fn = jl_gemv_tiles<TYPE, DUAL, RMS, PACKED, THREADS, SPT, SEGS, PART, ARGMAX, HALVES>;
    int per_cu = blocks_per_cu((const void *)fn, ctx->device, threads, lds);
    int total = p.seg_tile_begin[p.nseg];
    int grid = ctx->compute_units * per_cu;
    if (grid > total) grid = total;
    if (cells) {
        if (grid > *cells) return JL_NO_CELLS_FORM;   // more workgroups than the caller has cells for
        *cells = grid;
    }
    hipLaunchKernelGGL(fn, dim3(grid), dim3(threads), lds, ctx->stream, p.w[0], p.w_up, p.x, total, p.seg_rows[0], grid, p.S, p.row_bytes,
                       p.Sp | (p.R << 10) | (p.nseg << 20), p.rms_w, p);
    JL_HIP(hipGetLastError());
    return JL_OK;
}

// The 256-thread fixed-geometry instance of the three main types for rows padded to Sp slices of
// 64 columns, `full`: every slice is one of the row's (else the row is shorter: 3072 columns are 48
// of 64 slices, 5120 are 80 of 128).  -1: no instance for this Sp.
template <int TYPE, bool DUAL, bool RMS, bool SEGS, int SP>
int launch_fixed_sp(jl_context *ctx, const GemvParams &p, int lds, bool full) {
    return full ? launch_tiles_of<TYPE, DUAL, RMS, false, 256, SP, SEGS, false>(ctx, p, 256, lds)
                : launch_tiles_of<TYPE, DUAL, RMS, false, 256, SP, SEGS, true>(ctx, p, 256, lds);
}
template <int TYPE, bool DUAL, bool RMS, bool SEGS>
int launch_fixed(jl_context *ctx, const GemvParams &p, int lds, bool full) {
    switch (p.Sp) {
        case 16: return launch_fixed_sp<TYPE, DUAL, RMS, SEGS, 16>(ctx, p, lds, full);
        case 32: return launch_fixed_sp<TYPE, DUAL, RMS, SEGS, 32>(ctx, p, lds, full);
        case 64: return launch_fixed_sp<TYPE, DUAL, RMS, SEGS, 64>(ctx, p, lds, full);
        case 128: return launch_fixed_sp<TYPE, DUAL, RMS, SEGS, 128>(ctx, p, lds, full);
        default: return -1;
    }
}

// `fixed`: the launch meets the fixed-geometry form's conditions (whole tiles only in every
// weight).  The three main types have an instance for every variant at row lengths of 513 ... 8192
// columns and, in the 1024-thread form (plain and residual), up to 16384 -- and, a row taken as two
// half rows, up to 32768 (launched from jl_launch_gemv itself); the side types for whole rows of
// 2048, 4096 and (plain and residual) 8192 columns.
template <int TYPE, bool DUAL>
int launch_tiles(jl_context *ctx, const GemvParams &p, int threads, int lds, bool fixed, int *cells = nullptr) {
    // (side types: plain, residual and gate/up only -- the caller has refused the rest)
    constexpr bool kMain = is_main_type(TYPE);
    if (cells) {
        // the argmax form: one main-type weight, whole tiles of whole in-wave rows of 2048 or 4096
        // columns, stored (not accumulated) outputs
        if constexpr (kMain && !DUAL) {
            if (fixed && threads == 256 && p.S == p.Sp && p.nseg == 1 && !p.xq && p.epilogue == JL_STORE) {
                if (p.Sp == 32)
                    return p.rms_w ? launch_tiles_of<TYPE, false, true, false, 256, 32, false, false, true>(ctx, p, 256, lds, cells)
                                   : launch_tiles_of<TYPE, false, false, false, 256, 32, false, false, true>(ctx, p, 256, lds, cells);
                if (p.Sp == 64)
                    return p.rms_w ? launch_tiles_of<TYPE, false, true, false, 256, 64, false, false, true>(ctx, p, 256, lds, cells)
                                   : launch_tiles_of<TYPE, false, false, false, 256, 64, false, false, true>(ctx, p, 256, lds, cells);
            }
        }
        return JL_NO_CELLS_FORM;
    }
    if constexpr (kMain) {
        if (p.xq) return launch_tiles_of<TYPE, DUAL, false, true>(ctx, p, threads, lds);
    }
    const bool full = fixed && p.S == p.Sp;
    if constexpr (kMain) {
        if (fixed && threads == 256) {
            int st;
            // (the RMS-folding projections are q|k|v, gate/up and the vocabulary: rows of dim columns)
            if constexpr (DUAL) {
                st = p.rms_w ? launch_fixed<TYPE, true, true, false>(ctx, p, lds, full)
                             : launch_fixed<TYPE, true, false, false>(ctx, p, lds, full);
            } else if (p.nseg > 1) {
                st = p.rms_w ? launch_fixed<TYPE, false, true, true>(ctx, p, lds, full)
                             : launch_fixed<TYPE, false, false, true>(ctx, p, lds, full);
            } else {
                st = p.rms_w ? launch_fixed<TYPE, false, true, false>(ctx, p, lds, full)
                             : launch_fixed<TYPE, false, false, false>(ctx, p, lds, full);
            }
            if (st != -1) return st;
        }
        if (p.rms_w) return launch_tiles_of<TYPE, DUAL, true>(ctx, p, threads, lds);
    } else {
        if (full && threads == 256) {
            if (p.Sp == 32) return launch_tiles_of<TYPE, DUAL, false, false, 256, 32>(ctx, p, threads, lds);
            if (p.Sp == 64) return launch_tiles_of<TYPE, DUAL, false, false, 256, 64>(ctx, p, threads, lds);
            if constexpr (!DUAL) {
                if (p.Sp == 128) return launch_tiles_of<TYPE, false, false, false, 256, 128>(ctx, p, threads, lds);
            }
        }
    }
    if constexpr (!DUAL) {
        if (threads == kWideThreads) {
            if (fixed && p.Sp == 256 && p.nseg == 1) {
                return p.S == p.Sp ? launch_tiles_of<TYPE, false, false, false, kWideThreads, 256>(ctx, p, threads, lds)
                                   : launch_tiles_of<TYPE, false, false, false, kWideThreads, 256, false, true>(ctx, p, threads, lds);
            }
            return launch_tiles_of<TYPE, false, false, false, kWideThreads>(ctx, p, threads, lds);
        }
    }
    return launch_tiles_of<TYPE, DUAL, false>(ctx, p, threads, lds);
}

template <int TYPE>
int launch_generic(jl_context *ctx, const jl_weight *w, const jl_weight *w_up, const float *x,
                   float *out, int epilogue) {
    int rows = (int)w->rows;
    hipLaunchKernelGGL(jl_gemv_generic<TYPE>, dim3((rows + 3) / 4), dim3(256), 0, ctx->stream,
                       w->blocks, w_up ? w_up->blocks : nullptr, x, out, rows, (int)w->cols, epilogue);
    JL_HIP(hipGetLastError());
    return JL_OK;
}

}  // namespace


int jl_launch_gemv(jl_context *ctx, const jl_weight *const *w, int nseg, float *const *outs,
                   const jl_weight *w_up, const float *x, int epilogue, const jl_rms *rms, const jl_q8x *xq,
                   jl_best_cells *cells) {
    const int type = w[0]->type;
    const int n = (int)w[0]->cols;
    const int row_bytes = n / jl_block_elems(type) * jl_block_bytes(type);
    if (cells && !is_main_type(type)) return JL_NO_CELLS_FORM;
    if (xq && !jl_has_fused_kernels(type)) {
        return jl_fail(JL_ERR_UNSUPPORTED, "no packed-activation kernel for a %s weight", jl_type_name(type));
    }
    if (!jl_has_fused_kernels(type)) {
        if (nseg != 1 || rms) {
            return jl_fail(JL_ERR_UNSUPPORTED, "no fused q|k|v or RMS-folding single-token kernel for a %s weight "
                                               "(plain, residual and gate/up projections only)", jl_type_name(type));
        }
        // Q6_K and Q5_K go on to the tile kernel when the shape allows, the rest have the
        // one-wave-per-row kernels
        if (!is_side_type(type)) return jl_launch_gemv_direct(ctx, w[0], w_up, x, outs[0], epilogue);
    }

    const bool dual = w_up != nullptr;
    // bytes a thread brings in per tile
    const int slice = type == JL_Q8_0 ? 68 : type == JL_Q6_K ? 64 : is_side_type(type) ? 48 : 36;
    // Rows of 16 448 .. 32 768 columns, plain and residual projections of the three main types: the
    // weight seen as [2 rows x n / 2] (the kernel's HALVES form); a half row is whole blocks, a tile
    // -- four half rows, two rows -- whole 16-byte pieces.
    if (is_main_type(type) && !dual && !rms && !xq && !cells && nseg == 1 && n > 16384 && n <= 32768 &&
        n % 128 == 0 && (n / 2) % jl_block_elems(type) == 0 && w[0]->rows % 2 == 0 && ((uintptr_t)x & 15) == 0 &&
        ((uintptr_t)w[0]->blocks & 15) == 0 && ((int64_t)2 * row_bytes) % 16 == 0) {
        GemvParams h{};
        h.nseg = 1;
        h.w[0] = w[0]->blocks;
        h.out[0] = outs[0];
        h.seg_rows[0] = 2 * (int)w[0]->rows;
        h.seg_tile_begin[1] = (int)w[0]->rows / 2;
        h.x = x;
        h.n = n;
        h.S = n / 128;
        h.Sp = 256;
        h.R = 4;
        h.row_bytes = row_bytes / 2;
        h.epilogue = epilogue;
        const int lds = kPartialBytes + kStages * kWideThreads * slice;
        switch (type) {
            case JL_Q8_0: return launch_tiles_of<JL_Q8_0, false, false, false, kWideThreads, 256, false, true, false, true>(ctx, h, kWideThreads, lds);
            case JL_Q4_0: return launch_tiles_of<JL_Q4_0, false, false, false, kWideThreads, 256, false, true, false, true>(ctx, h, kWideThreads, lds);
            default: return launch_tiles_of<JL_Q4_K, false, false, false, kWideThreads, 256, false, true, false, true>(ctx, h, kWideThreads, lds);
        }
    }
    bool fast = (n % 64 == 0) && (n / 64 <= 256) &&
                (xq ? (((uintptr_t)xq->quants & 15) == 0 && ((uintptr_t)xq->scales & 7) == 0 &&
                       ((uintptr_t)xq->sums & 7) == 0)
                    : (((uintptr_t)x & 15) == 0));
    int S = n / 64, Sp = 0, R = 0, half_rows = 0;
    if (fast) {
        Sp = next_pow2(S);
        // Rows of more than 128 slices (8192 columns): a workgroup of 256 threads would hold one
        // row per tile and stage the whole activation vector -- more bytes than its tiles -- for
        // it, at one workgroup per compute unit for the LDS that takes.  Sixteen waves share the
        // staged vector instead (plain and residual projections; the other variants keep 256).
        // (when its LDS fits: Q8_0 rows of more than 15 360 columns do not)
        const bool wide = Sp == 256 && !dual && !rms && !xq && tile_lds_bytes(kWideThreads, slice, S, is_side_type(type)) <= 160 * 1024;
        R = (wide ? kWideThreads : 256) / Sp;
        half_rows = dual ? R / 2 : R;
        if (half_rows < 1) fast = false;
        else if (((int64_t)half_rows * row_bytes) % 16 != 0) fast = false;
    }
    for (int i = 0; fast && i < nseg; i++) {
        if (((uintptr_t)w[i]->blocks & 15) != 0) fast = false;
        // the last tile is brought in by whole 16-byte loads too: a weight whose bytes do not end on
        // a 16-byte boundary (a few odd rows of a 64- or 128-column weight) would lose its tail
        if ((w[i]->rows * (int64_t)row_bytes) % 16 != 0) fast = false;
    }
    if (w_up && ((uintptr_t)w_up->blocks & 15) != 0) fast = false;

    if (cells && !fast) return JL_NO_CELLS_FORM;
    if (!fast && xq) {
        return jl_fail(JL_ERR_UNSUPPORTED,
                       "no packed-activation kernel for a row length of %d (a multiple of 64 up to %d "
                       "and aligned operands are needed)", n, dual ? 8192 : 16384);
    }
    if (!fast && rms) {
        return jl_fail(JL_ERR_UNSUPPORTED,
                       "no RMS-folding projection kernel for a row length of %d (a multiple of 64 up to "
                       "%d and 16-byte aligned operands are needed)", n, dual ? 8192 : 16384);
    }
    if (rms && ((uintptr_t)rms->weights & 15) != 0) {
        return jl_fail(JL_ERR_UNSUPPORTED, "the RMS weights must be 16-byte aligned");
    }
    if (is_side_type(type)) {
        // measured: the tile kernel is the faster one from rows of 2048 columns and 2 MB of weights
        // (by up to 1.7 x on the vocabulary and feed-forward projections); below that the two are
        // within a few tenths of a microsecond of each other and the one-wave-per-row kernel stays
        if (!fast || n < 2048 || w[0]->bytes * (dual ? 2 : 1) < ((int64_t)2 << 20))
            return jl_launch_gemv_direct(ctx, w[0], w_up, x, outs[0], epilogue);
    }
    if (!fast) {
        for (int i = 0; i < nseg; i++) {
            int st;
            switch (type) {
                case JL_Q8_0: st = launch_generic<JL_Q8_0>(ctx, w[i], w_up, x, outs[i], epilogue); break;
                case JL_Q4_0: st = launch_generic<JL_Q4_0>(ctx, w[i], w_up, x, outs[i], epilogue); break;
                case JL_Q4_K: st = launch_generic<JL_Q4_K>(ctx, w[i], w_up, x, outs[i], epilogue); break;
                default:
                    return jl_fail(JL_ERR_UNSUPPORTED,
                                   "no single-token projection kernel for a ggml type %d weight", type);
            }
            if (st != JL_OK) return st;
        }
        return JL_OK;
    }

    GemvParams p{};
    p.nseg = nseg;
    int tiles = 0;
    for (int i = 0; i < nseg; i++) {
        p.w[i] = w[i]->blocks;
        p.out[i] = outs[i];
        p.seg_rows[i] = (int)w[i]->rows;
        p.seg_tile_begin[i] = tiles;
        tiles += ((int)w[i]->rows + half_rows - 1) / half_rows;
    }
    p.seg_tile_begin[nseg] = tiles;
    p.w_up = w_up ? w_up->blocks : nullptr;
    p.x = x;
    p.n = n;
    p.S = S;
    p.Sp = Sp;
    p.R = R;
    p.row_bytes = row_bytes;
    p.epilogue = epilogue;
    if (xq) {
        p.xq = xq->quants;
        p.xq_scales = xq->scales;
        p.xq_sums = xq->sums;
    }
    if (rms) {
        p.rms_w = rms->weights;
        p.rms_scale = rms->scale;
        p.rms_eps = rms->eps;
    }
    if (cells) {
        p.best_value = cells->value;
        p.best_index = cells->index;
    }

    const int threads = (R * Sp + 63) / 64 * 64;
    const int lds = tile_lds_bytes(threads, slice, S, is_side_type(type));
    // (whole tiles only; `full`: rows of exactly Sp slices as well)
    bool fixed = R * Sp == threads;
    for (int i = 0; i < nseg; i++) fixed = fixed && w[i]->rows % half_rows == 0;

    if (cells) {
        if (dual) return JL_NO_CELLS_FORM;
        switch (type) {
            case JL_Q8_0: return launch_tiles<JL_Q8_0, false>(ctx, p, threads, lds, fixed, &cells->count);
            case JL_Q4_0: return launch_tiles<JL_Q4_0, false>(ctx, p, threads, lds, fixed, &cells->count);
            case JL_Q4_K: return launch_tiles<JL_Q4_K, false>(ctx, p, threads, lds, fixed, &cells->count);
            default: return JL_NO_CELLS_FORM;
        }
    }
    switch (type) {
        case JL_Q8_0:
            return dual ? launch_tiles<JL_Q8_0, true>(ctx, p, threads, lds, fixed)
                        : launch_tiles<JL_Q8_0, false>(ctx, p, threads, lds, fixed);
        case JL_Q4_0:
            return dual ? launch_tiles<JL_Q4_0, true>(ctx, p, threads, lds, fixed)
                        : launch_tiles<JL_Q4_0, false>(ctx, p, threads, lds, fixed);
        case JL_Q4_K:
            return dual ? launch_tiles<JL_Q4_K, true>(ctx, p, threads, lds, fixed)
                        : launch_tiles<JL_Q4_K, false>(ctx, p, threads, lds, fixed);
        case JL_Q6_K:
            return dual ? launch_tiles<JL_Q6_K, true>(ctx, p, threads, lds, fixed)
                        : launch_tiles<JL_Q6_K, false>(ctx, p, threads, lds, fixed);
        case JL_Q5_K:
            return dual ? launch_tiles<JL_Q5_K, true>(ctx, p, threads, lds, fixed)
                        : launch_tiles<JL_Q5_K, false>(ctx, p, threads, lds, fixed);
        case JL_Q4_1:
            return dual ? launch_tiles<JL_Q4_1, true>(ctx, p, threads, lds, fixed)
                        : launch_tiles<JL_Q4_1, false>(ctx, p, threads, lds, fixed);
        case JL_Q5_0:
            return dual ? launch_tiles<JL_Q5_0, true>(ctx, p, threads, lds, fixed)
                        : launch_tiles<JL_Q5_0, false>(ctx, p, threads, lds, fixed);
        case JL_IQ4_XS:
            return dual ? launch_tiles<JL_IQ4_XS, true>(ctx, p, threads, lds, fixed)
                        : launch_tiles<JL_IQ4_XS, false>(ctx, p, threads, lds, fixed);
        default:
            return jl_fail(JL_ERR_UNSUPPORTED,
                           "no single-token projection kernel for a ggml type %d weight", type);
    }
}
