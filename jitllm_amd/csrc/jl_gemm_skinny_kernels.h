// Batched decode (at most 64 activation rows; up to 511 as row blocks of 32 where the launcher
// prices that cheaper than the tiled kernels): C = X . [W0 | W1 | ...]^T streamed at HBM speed.
//
// Replaces the reference's tiled batched-row kernels (matrixVectorTiledBatchQ4_0 / Q4_K,
// J/backend/tornado/kernels/TransformerComputeKernelsQ4_0.java:1205-1292,
// TransformerComputeKernelsQ4_K.java:1120-1221, driven by QuantizedBatchProjections.java:76-309).
//
// With so few rows the call is bound by reading the weights once, exactly like the single-token
// matrix-vector kernels, so this kernel has their shape: a workgroup walks tiles of 16 weight rows,
// a tile is copied into an LDS ring by LDS-DMA while the previous one is computed, and a thread
// owns one 64-column slice of its weight row.  What differs is the arithmetic: the thread turns its
// slice into eight fp16 fragments of eight consecutive columns in registers, and a wave (16 rows x
// 4 slices) multiplies them with the matching activation fragments on v_mfma_f32_16x16x32_f16.  The
// MFMA sums over 32 "k slots"; slot (g, e) of MFMA i is column 64 (slice of lane group g) + 8 i + e,
// the same for both operands, so no data crosses lanes.  The activations are the MFMA's row operand
// and the weights its column operand: a lane's four results belong to the weight row it decoded.
//
// Q8_0 / Q4_0 fragments are the decoded weights (q - bias) * d rounded once to fp16.  Q4_K fragments
// are the exact integers sc * q (at most 945): a wave's four slices are the four nibble pairs of one
// super-block, so d and dmin are common to everything its eight MFMAs add up and are applied to
// their result -- the reference's blockDot formulation, TransformerComputeKernelsQ4_K.java:270-373 --
// and the minimum term sum_j m_j * (sum of x over sub-block j) is a ninth MFMA over the sub-blocks'
// activation sums.  That is 1.4 vector instructions per weight instead of 3, and no weight is
// rounded at all.
//
// The activation fragments (read as fp32 and rounded to fp16 by the kernel itself) depend on the
// slice only and stay in registers for the whole kernel.  A wave's result is a partial sum over its
// 256 columns; two waves of their own fold the compute waves' partials through LDS two tiles later
// and apply the epilogue (one row block each when there are two), rows wider than the workgroup's
// span are cut across workgroups and folded, inside the launch, by the workgroup that arrives
// last.  The two compute waves of a SIMD run half a tile apart: one decodes while the other
// multiplies.  Calls of more than 32 rows run as row blocks of up to 32 that share the chip (two
// halves at 33..64 rows); the blocks walk the same tiles at about the same time, so the later
// readers of a tile may find it in the L2 of their XCD.
//
// This file is compiled twice: jl_gemm_skinny.hip includes it for fp32 activations, and
// jl_gemm_skinny_x16.hip for binary16 ones (JL_SKINNY_XH; the entry point's name is
// JL_SKINNY_ENTRY) -- two translation units, so that the two sets of instances build side by side.
#include <stdlib.h>

#include "jl_device.h"
#include "jl_internal.h"

namespace {

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef _Float16 h2 __attribute__((ext_vector_type(2)));
typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(1))) const void gvoid;
typedef __attribute__((address_space(3))) void lvoid;

constexpr int kMaxSeg = 8;
// The weight stream is read once: its LDS-DMA loads are marked non-temporal (bit 1 of the cache
// policy).  Measured per layer (four calls in turn, graph replays, one box): Q4_K at 8B shapes
// 48.6 / 56.6 / 75.6 / 99.0 -> 46.2 / 54.6 / 74.8 / 98.4 us at 8 / 16 / 32 / 64 rows, Q8_0 at Llama-3.2-1B
// shapes 38.8 / 40.6 / 46.1 / 53.0 -> 34.9 / 37.5 / 44.4 / 51.5 us.  A call timed on its own gains only
// where it reads two weights in turn (gate/up); the rest comes from what the stream no longer
// pushes out of the caches between one call and the next.
constexpr int kStreamNonTemporal = 2;
constexpr int kGroup = 16;  // weight rows per tile: the MFMA's row count

// (A field added in the middle of this struct -- twelve bytes that moved the ones behind it -- cost
// every call 0.6 us, measured; an order with what the copy waves need first gained nothing.  New
// fields go to the end.)
struct SkinnyParams {
    const uint8_t *w[kMaxSeg];
    int seg_rows[kMaxSeg];
    int seg_group_begin[kMaxSeg + 1];  // first row group of each weight; [nseg] = all groups
    int seg_col_begin[kMaxSeg];        // first output column of each weight
    int nseg;
    const uint8_t *w_up;      // JL_SWIGLU: the up weight (a group is 8 gate rows + 8 up rows)
    const float *X;           // [rows x k] activations: fp32, or (JL_SKINNY_XH) binary16 behind the same pointer
    float *C;
    float *planes;            // Z > 1: [Z][row blocks][groups][64 lanes] x 4 partial sums, as the fold's lanes hold them
    uint32_t *arrivals;       // Z > 1: one counter per (set of workgroups that share their groups, row block); all 0 between calls
    int rows;                 // active activation rows
    int k;
    int64_t ldo, col_offset;
    int epilogue;
    int row_bytes;
    int Ss;                   // 64-column slices one workgroup spans (a multiple of 4, at most 32)
    int Z;                    // spans per row
    int span_bytes;           // bytes of a weight row inside one span
    int stages;               // depth of the tile ring
    int row_blocks;           // gridDim.y: blocks of 16 NBB activation rows, each on its own workgroups
    int c_f16;                // binary16 activations, JL_SWIGLU only: C holds binary16 values, ldo and col_offset count them
};

#define JL_WAIT_VM(N) \
    __builtin_amdgcn_s_waitcnt(((N)&0xF) | (((N) >> 4) << 14) | (0x7 << 4) | (0xF << 8))

// s_waitcnt vmcnt(n) for a run-time n (the instruction takes an immediate)
__device__ __forceinline__ void wait_vm(int n) {
    switch (n) {
#define C(i) case i: JL_WAIT_VM(i); break;
        C(0) C(1) C(2) C(3) C(4) C(5) C(6) C(7) C(8) C(9) C(10) C(11) C(12) C(13) C(14) C(15)
        C(16) C(17) C(18) C(19) C(20) C(21) C(22) C(23) C(24) C(25) C(26) C(27) C(28) C(29) C(30)
        C(31) C(32) C(33) C(34) C(35) C(36) C(37) C(38) C(39) C(40) C(41) C(42) C(43) C(44) C(45)
        C(46) C(47) C(48) C(49) C(50) C(51) C(52) C(53) C(54) C(55) C(56) C(57) C(58) C(59) C(60)
        C(61) C(62)
#undef C
        default: JL_WAIT_VM(63); break;
    }
}

// ---- LDS access by hand (the compiler would drain the LDS-DMA ring before any LDS access it sees)

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

__device__ __forceinline__ void lds_read_q4k(uint32_t hdr, uint32_t qs, uint4 &h, uint4 &q0, uint4 &q1) {
    asm volatile(
        "ds_read_b128 %0, %3\n\tds_read_b128 %1, %4\n\tds_read_b128 %2, %4 offset:16\n\t"
        "s_waitcnt lgkmcnt(0)"
        : "=&v"(h), "=&v"(q0), "=&v"(q1) : "v"(hdr), "v"(qs) : "memory");
}

// N 16-byte reads at consecutive 16-byte offsets from `addr` (16-byte aligned), one wait.
template <int N>
__device__ __forceinline__ void lds_read_x4(uint32_t addr, u32x4 (&v)[N]) {
#pragma unroll
    for (int i = 0; i < N; i++) asm volatile("ds_read_b128 %0, %1 offset:%2" : "=&v"(v[i]) : "v"(addr), "n"(16 * i) : "memory");
}
// N dword reads at consecutive offsets from `addr` (4-byte aligned)
template <int N>
__device__ __forceinline__ void lds_read_x1(uint32_t addr, uint32_t (&v)[N]) {
#pragma unroll
    for (int i = 0; i < N; i++) asm volatile("ds_read_b32 %0, %1 offset:%2" : "=&v"(v[i]) : "v"(addr), "n"(4 * i) : "memory");
}
// The wait behind reads issued without one; the values pass through it so that no use moves ahead.
template <typename T, int N>
__device__ __forceinline__ void lds_landed(T (&v)[N]) {
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
#pragma unroll
    for (int i = 0; i < N; i++) {
        T t = v[i];
        asm volatile("" : "+v"(t));
        v[i] = t;
    }
}

// Partial sums that travel from one workgroup to another inside a launch: stores written through to
// device scope and loads that are served from there (the sc1 cache policy; what the compiler emits
// for relaxed atomic accesses at agent scope), 16 bytes per lane.  The eight XCDs' L2 caches are
// not kept coherent by hardware, and the by-the-book alternative -- plain accesses between a
// release fence and an acquire fence at agent scope -- writes back and invalidates a whole L2 on
// every fence (measured here: 10-20 us a call).  The load does not wait for its data: the caller
// waits (s_waitcnt vmcnt) in a statement that every destination register passes through.
__device__ __forceinline__ void agent_store_f4(floatx4 *p, floatx4 v) {
    // (a store of more than 8 bytes reads its data registers for two more cycles: the wait states
    // the compiler would place before a write of those registers, had it emitted the store itself)
    asm volatile("global_store_dwordx4 %0, %1, off sc1\n\ts_nop 1" : : "v"(p), "v"(v) : "memory");
}
__device__ __forceinline__ floatx4 agent_load_f4(const floatx4 *p) {
    floatx4 v;
    asm volatile("global_load_dwordx4 %0, %1, off sc1" : "=&v"(v) : "v"(p) : "memory");
    return v;
}
__device__ __forceinline__ void vm_drained() { asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); }

// Never hand an MFMA result straight to this: the matrix pipe does not interlock with an LDS store
// that reads its destination registers, and the compiler's hazard pass cannot see inside inline
// assembly.  Callers pass values that went through ordinary vector arithmetic first.
__device__ __forceinline__ void lds_write_f4(uint32_t addr, floatx4 v) {
    asm volatile("ds_write_b128 %0, %1\n\ts_waitcnt lgkmcnt(0)"
                 : : "v"(addr), "v"(v) : "memory");
}

__device__ __forceinline__ floatx4 lds_read_f4(uint32_t addr) {
    floatx4 v;
    asm volatile("ds_read_b128 %0, %1\n\ts_waitcnt lgkmcnt(0)" : "=&v"(v) : "v"(addr) : "memory");
    return v;
}

// ---- slice decode: raw block bytes -> eight fp16 fragments of eight consecutive columns ---------
//
// A byte b in 0..255 under the exponent byte 0x64 is the fp16 number 1024 + b, exactly; a packed
// subtract recentres it and a packed multiply applies the block scale.  Each product is exact
// before its one rounding, so a decoded weight is the host's float decode rounded once to fp16.

__device__ __forceinline__ h2 bytes_to_h2(uint32_t v, uint32_t sel) {
    return __builtin_bit_cast(h2, __builtin_amdgcn_perm(v, 0x64646464u, sel));
}

// eight bytes (two dwords, already in 0..255 offset form) -> (byte - bias) * d
__device__ __forceinline__ half8 frag_scaled(uint32_t q0, uint32_t q1, h2 bias, h2 d) {
    h2 a = (bytes_to_h2(q0, 0x00050004u) - bias) * d;
    h2 b = (bytes_to_h2(q0, 0x00070006u) - bias) * d;
    h2 c = (bytes_to_h2(q1, 0x00050004u) - bias) * d;
    h2 e = (bytes_to_h2(q1, 0x00070006u) - bias) * d;
    return half8{a[0], a[1], b[0], b[1], c[0], c[1], e[0], e[1]};
}

// eight nibbles (two dwords of bytes 0..15) -> the exact integers q * sc: (1024 + q) * sc - 1024 sc
// in one fused step, so the only rounding would be that of the (exact) result
__device__ __forceinline__ half8 frag_times(uint32_t q0, uint32_t q1, h2 sc, h2 off) {
    h2 a = __builtin_elementwise_fma(bytes_to_h2(q0, 0x00050004u), sc, off);
    h2 b = __builtin_elementwise_fma(bytes_to_h2(q0, 0x00070006u), sc, off);
    h2 c = __builtin_elementwise_fma(bytes_to_h2(q1, 0x00050004u), sc, off);
    h2 e = __builtin_elementwise_fma(bytes_to_h2(q1, 0x00070006u), sc, off);
    return half8{a[0], a[1], b[0], b[1], c[0], c[1], e[0], e[1]};
}

// What a Q4_K slice needs beside its fragments: the super-block's d and dmin (applied to the MFMA
// results) and the two sub-blocks' minimums as the k slots of the minimum MFMA.
struct Q4KTail {
    float d, dmin;
    half8 mins;   // {m0, m0, m1, m1, 0, 0, 0, 0}: each minimum meets its sub-block's activation sum as hi + lo
};

// Bytes of 256 columns of a row (four slices): every type's blocks tile 256 columns exactly.
constexpr int quad_bytes(int type) {
    return type == JL_Q8_0 ? 272 : type == JL_Q4_0 ? 144 : type == JL_Q4_K ? 144 : type == JL_Q6_K ? 210
           : type == JL_Q5_K ? 176 : type == JL_Q4_1 ? 160 : type == JL_Q5_0 ? 176 : type == JL_IQ4_XS ? 136 : 0;
}
// Types whose 256-column block has one scale for everything a wave's MFMAs add up: the fragments
// hold small integers (sub-block scale x quant) and the block's d multiplies the MFMA result.
template <int TYPE> constexpr bool kPostScale = TYPE == JL_Q4_K || TYPE == JL_Q5_K || TYPE == JL_Q6_K || TYPE == JL_IQ4_XS;
// Types with an additive term per 32 columns (a minimum), folded in by one more MFMA against the
// activations' sums over those 32 columns.
template <int TYPE> constexpr bool kHasMins = TYPE == JL_Q4_K || TYPE == JL_Q5_K || TYPE == JL_Q4_1;

// The scales and minimums of sub-blocks 2 pair and 2 pair + 1 of a Q4_K / Q5_K header (d, dmin, 12
// packed bytes: h.y, h.z, h.w), each scale as a pair of equal fp16 values, the minimums as the k
// slots of the minimum MFMA.  Sub-blocks 0..3 keep them in the low six bits of bytes j and j + 4,
// sub-blocks 4..7 in the nibbles of byte j + 4 with bits 4..5 in the top bits of bytes j - 4 and j
// (Q4_KFloatTensor.getScaleK4 / getMinK4, J/tensor/standard/Q4_KFloatTensor.java:68-85).
__device__ __forceinline__ void k_scales(const uint4 &h, int pair, h2 &s0, h2 &s1, Q4KTail &tail) {
    tail.d = jl_half_bits_to_float(h.x);
    tail.dmin = jl_half_bits_to_float(h.x >> 16);
    const int sh = 16 * (pair & 1);
    const uint32_t a = h.y >> sh, b = h.z >> sh, c = h.w >> sh;
    const uint32_t sc2 = pair < 2 ? (a & 0x3F3Fu) : ((c & 0x0F0Fu) | ((a >> 2) & 0x3030u));
    const uint32_t mn2 = pair < 2 ? (b & 0x3F3Fu) : (((c >> 4) & 0x0F0Fu) | ((b >> 2) & 0x3030u));
    // small integers as fp16: bits 0x6400 | v are 1024 + v
    const h2 k1024 = {(_Float16)1024.f, (_Float16)1024.f};
    s0 = __builtin_bit_cast(h2, __builtin_amdgcn_perm(sc2, 0x64646464u, 0x00040004u)) - k1024;
    s1 = __builtin_bit_cast(h2, __builtin_amdgcn_perm(sc2, 0x64646464u, 0x00050005u)) - k1024;
    const h2 m01 = __builtin_bit_cast(h2, __builtin_amdgcn_perm(mn2, 0x64646464u, 0x00040004u)) - k1024;
    const h2 m11 = __builtin_bit_cast(h2, __builtin_amdgcn_perm(mn2, 0x64646464u, 0x00050005u)) - k1024;
    const _Float16 z = (_Float16)0.f;
    tail.mins = half8{m01[0], m01[1], m11[0], m11[1], z, z, z, z};
}

// a signed byte of `v` as a pair of equal fp16 values
__device__ __forceinline__ h2 sbyte_h2(uint32_t v, int byte) {
    const _Float16 f = (_Float16)(float)(int)(int8_t)(v >> (8 * byte));
    return h2{f, f};
}

// Decodes the 64-column slice `sl` of the tile row at LDS address `row`.
template <int TYPE>
__device__ __forceinline__ void decode_slice(uint32_t row, int sl, half8 (&f)[8], Q4KTail &tail) {
    if constexpr (TYPE == JL_Q8_0) {
        // 68 bytes: scale A | 32 quants A | scale B | 32 quants B
        uint32_t w[17];
        lds_read_17(row + sl * 68, w);
        const _Float16 dA = __builtin_bit_cast(_Float16, (unsigned short)(w[0] & 0xFFFF));
        const _Float16 dB = __builtin_bit_cast(_Float16, (unsigned short)(w[8] >> 16));
        const h2 bias = {(_Float16)1152.f, (_Float16)1152.f};
        const h2 a2 = {dA, dA}, b2 = {dB, dB};
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const uint32_t q0 = __builtin_amdgcn_alignbit(w[2 * i + 1], w[2 * i], 16);
            const uint32_t q1 = __builtin_amdgcn_alignbit(w[2 * i + 2], w[2 * i + 1], 16);
            f[i] = frag_scaled(q0 ^ 0x80808080u, q1 ^ 0x80808080u, bias, a2);
            f[4 + i] = frag_scaled(w[9 + 2 * i] ^ 0x80808080u, w[10 + 2 * i] ^ 0x80808080u, bias, b2);
        }
    } else if constexpr (TYPE == JL_Q4_0) {
        // 36 bytes: scale A | 16 nibble bytes A | scale B | 16 nibble bytes B; element i < 16 of a
        // block is the low nibble of byte i, element 16 + i the high nibble
        uint32_t w[9];
        lds_read_9(row + sl * 36, w);
        const _Float16 dA = __builtin_bit_cast(_Float16, (unsigned short)(w[0] & 0xFFFF));
        const _Float16 dB = __builtin_bit_cast(_Float16, (unsigned short)(w[4] >> 16));
        const h2 bias = {(_Float16)1032.f, (_Float16)1032.f};
        const h2 a2 = {dA, dA}, b2 = {dB, dB};
        uint32_t qa[4], qb[4];
#pragma unroll
        for (int i = 0; i < 4; i++) {
            qa[i] = __builtin_amdgcn_alignbit(w[i + 1], w[i], 16);
            qb[i] = w[5 + i];
        }
#pragma unroll
        for (int i = 0; i < 2; i++) {
            f[i] = frag_scaled(qa[2 * i] & 0x0F0F0F0Fu, qa[2 * i + 1] & 0x0F0F0F0Fu, bias, a2);
            f[2 + i] = frag_scaled((qa[2 * i] >> 4) & 0x0F0F0F0Fu, (qa[2 * i + 1] >> 4) & 0x0F0F0F0Fu, bias, a2);
            f[4 + i] = frag_scaled(qb[2 * i] & 0x0F0F0F0Fu, qb[2 * i + 1] & 0x0F0F0F0Fu, bias, b2);
            f[6 + i] = frag_scaled((qb[2 * i] >> 4) & 0x0F0F0F0Fu, (qb[2 * i + 1] >> 4) & 0x0F0F0F0Fu, bias, b2);
        }
    } else if constexpr (TYPE == JL_Q5_K) {
        // Q4_K's layout with a fifth bit per weight (fp16 d, dmin | 12 scale bytes | qh[32] |
        // qs[128], J/tensor/standard/Q5_KFloatTensor.java:78-122): bit 2 pair of qh[l] tops the low
        // nibble of qs[32 pair + l], bit 2 pair + 1 the high one.  sc q is at most 63 x 31: exact.
        const uint32_t sb = row + (sl >> 2) * 176;
        const int pair = sl & 3;
        u32x4 r[3], q[2];
        lds_read_x4(sb, r);                       // header, the 32 fifth-bit bytes
        lds_read_x4(sb + 48 + pair * 32, q);
        lds_landed(r);
        lds_landed(q);
        h2 s0, s1;
        k_scales(uint4{r[0].x, r[0].y, r[0].z, r[0].w}, pair, s0, s1, tail);
        const h2 o0 = s0 * h2{(_Float16)-1024.f, (_Float16)-1024.f};
        const h2 o1 = s1 * h2{(_Float16)-1024.f, (_Float16)-1024.f};
        const uint32_t qs[8] = {q[0].x, q[0].y, q[0].z, q[0].w, q[1].x, q[1].y, q[1].z, q[1].w};
        const uint32_t qh[8] = {r[1].x, r[1].y, r[1].z, r[1].w, r[2].x, r[2].y, r[2].z, r[2].w};
        uint32_t lo[8], hi[8];
#pragma unroll
        for (int j = 0; j < 8; j++) {
            const uint32_t hb = qh[j] >> (2 * pair);
            lo[j] = (qs[j] & 0x0F0F0F0Fu) | ((hb & 0x01010101u) << 4);
            hi[j] = ((qs[j] >> 4) & 0x0F0F0F0Fu) | ((hb & 0x02020202u) << 3);
        }
#pragma unroll
        for (int i = 0; i < 4; i++) {
            f[i] = frag_times(lo[2 * i], lo[2 * i + 1], s0, o0);
            f[4 + i] = frag_times(hi[2 * i], hi[2 * i + 1], s1, o1);
        }
    } else if constexpr (TYPE == JL_Q6_K) {
        // A quarter (h, upper) of a super-block (ql[128] | qh[64] | 16 signed scales | fp16 d,
        // J/tensor/standard/Q6_KFloatTensor.java:66-122): element l < 32 is nibble `upper` of
        // ql[64 h + l] under bits 4 upper .. + 1 of qh[32 h + l], element 32 + l nibble `upper` of
        // ql[64 h + 32 + l] under bits 4 upper + 2 .. + 3 of the same qh byte; one scale per 16
        // elements; w = d sc (q - 32).  A fragment holds sc (q - 32), an integer of at most 4096 in
        // magnitude (rounded to fp16 only beyond 2048), and d multiplies the MFMA result.
        // Super-blocks are 210 bytes apart, so every other one starts two bytes off a dword: the
        // quarter is read as aligned dwords from two bytes before where that is needed and each
        // dword put together from its two neighbours with a funnel shift of 0 or 16 bits.
        const uint32_t sb = row + (sl >> 2) * 210;
        const int h = (sl >> 1) & 1, upper = sl & 1;
        const uint32_t off = sb & 2u, shift = off * 8;
        uint32_t wl[17], wh[9], sc2[2], d16[1];
        lds_read_x1(sb - off + 64 * h, wl);
        lds_read_x1(sb - off + 128 + 32 * h, wh);
        lds_read_x1(sb - off + 192 + 4 * (sl & 3), sc2);
        asm volatile("ds_read_u16 %0, %1" : "=&v"(d16[0]) : "v"(sb + 208) : "memory");
        lds_landed(wl);
        lds_landed(wh);
        lds_landed(sc2);
        lds_landed(d16);
        tail.d = jl_half_bits_to_float(d16[0]);
        tail.dmin = 0.f;
        const uint32_t scales = __builtin_amdgcn_alignbit(sc2[1], sc2[0], shift);
        const h2 bias = {(_Float16)1056.f, (_Float16)1056.f};
        const int shl = 4 * upper;
        uint32_t v0[8], v1[8];
#pragma unroll
        for (int j = 0; j < 8; j++) {
            const uint32_t ql0 = __builtin_amdgcn_alignbit(wl[j + 1], wl[j], shift);
            const uint32_t ql1 = __builtin_amdgcn_alignbit(wl[9 + j], wl[8 + j], shift);
            const uint32_t hb = __builtin_amdgcn_alignbit(wh[j + 1], wh[j], shift) >> shl;
            v0[j] = ((ql0 >> shl) & 0x0F0F0F0Fu) | ((hb & 0x03030303u) << 4);
            v1[j] = ((ql1 >> shl) & 0x0F0F0F0Fu) | ((hb & 0x0C0C0C0Cu) << 2);
        }
#pragma unroll
        for (int i = 0; i < 4; i++) {
            f[i] = frag_scaled(v0[2 * i], v0[2 * i + 1], bias, sbyte_h2(scales, i >> 1));
            f[4 + i] = frag_scaled(v1[2 * i], v1[2 * i + 1], bias, sbyte_h2(scales, 2 + (i >> 1)));
        }
    } else if constexpr (TYPE == JL_Q4_1) {
        // 40 bytes: d, m | 16 nibble bytes, twice (J/tensor/standard/Q4_1FloatTensor.java:73-94);
        // w = d q + m.  The fragments hold d q rounded once; the minimums go through the extra MFMA
        // with the opposite sign of a K-quant's (dmin = -1).
        uint32_t w[10];
        lds_read_x1(row + sl * 40, w);
        lds_landed(w);
        const _Float16 dA = __builtin_bit_cast(_Float16, (unsigned short)(w[0] & 0xFFFF));
        const _Float16 mA = __builtin_bit_cast(_Float16, (unsigned short)(w[0] >> 16));
        const _Float16 dB = __builtin_bit_cast(_Float16, (unsigned short)(w[5] & 0xFFFF));
        const _Float16 mB = __builtin_bit_cast(_Float16, (unsigned short)(w[5] >> 16));
        const _Float16 z = (_Float16)0.f;
        tail.d = 1.f;
        tail.dmin = -1.f;
        tail.mins = half8{mA, mA, mB, mB, z, z, z, z};
        const h2 bias = {(_Float16)1024.f, (_Float16)1024.f};
        const h2 a2 = {dA, dA}, b2 = {dB, dB};
#pragma unroll
        for (int i = 0; i < 2; i++) {
            f[i] = frag_scaled(w[1 + 2 * i] & 0x0F0F0F0Fu, w[2 + 2 * i] & 0x0F0F0F0Fu, bias, a2);
            f[2 + i] = frag_scaled((w[1 + 2 * i] >> 4) & 0x0F0F0F0Fu, (w[2 + 2 * i] >> 4) & 0x0F0F0F0Fu, bias, a2);
            f[4 + i] = frag_scaled(w[6 + 2 * i] & 0x0F0F0F0Fu, w[7 + 2 * i] & 0x0F0F0F0Fu, bias, b2);
            f[6 + i] = frag_scaled((w[6 + 2 * i] >> 4) & 0x0F0F0F0Fu, (w[7 + 2 * i] >> 4) & 0x0F0F0F0Fu, bias, b2);
        }
    } else if constexpr (TYPE == JL_Q5_0) {
        // 44 bytes: d | 32 fifth bits | 16 nibble bytes, twice (J/tensor/standard/Q5_0FloatTensor.java:
        // 61-85); w = d (q - 16), bit i of the 32 tops element i.  Block A's fields sit two bytes off
        // the dwords (d | qh lo, qh hi | qs ..), block B's on them.
        uint32_t w[11];
        lds_read_x1(row + sl * 44, w);
        lds_landed(w);
        const _Float16 dA = __builtin_bit_cast(_Float16, (unsigned short)(w[0] & 0xFFFF));
        const _Float16 dB = __builtin_bit_cast(_Float16, (unsigned short)(w[5] >> 16));
        const h2 bias = {(_Float16)1040.f, (_Float16)1040.f};
        const h2 d2[2] = {h2{dA, dA}, h2{dB, dB}};
        const uint32_t qh[2] = {__builtin_amdgcn_alignbit(w[1], w[0], 16), w[6]};
        uint32_t qs[8];
#pragma unroll
        for (int j = 0; j < 4; j++) {
            qs[j] = __builtin_amdgcn_alignbit(w[2 + j], w[1 + j], 16);
            qs[4 + j] = w[7 + j];
        }
#pragma unroll
        for (int blk = 0; blk < 2; blk++) {
            uint32_t lo[4], hi[4];
#pragma unroll
            for (int j = 0; j < 4; j++) {
                const uint32_t q = qs[4 * blk + j];
                lo[j] = (q & 0x0F0F0F0Fu) | (jl_spread4(qh[blk] >> (4 * j)) << 4);
                hi[j] = ((q >> 4) & 0x0F0F0F0Fu) | (jl_spread4(qh[blk] >> (16 + 4 * j)) << 4);
            }
#pragma unroll
            for (int i = 0; i < 2; i++) {
                f[4 * blk + i] = frag_scaled(lo[2 * i], lo[2 * i + 1], bias, d2[blk]);
                f[4 * blk + 2 + i] = frag_scaled(hi[2 * i], hi[2 * i + 1], bias, d2[blk]);
            }
        }
    } else if constexpr (TYPE == JL_IQ4_XS) {
        // A quarter of a super-block (fp16 d | scales_h | scales_l[4] | qs[128],
        // J/tensor/standard/IQ4_XSFloatTensor.java:72-100): sub-blocks 2 q and 2 q + 1,
        // w = d (ls - 32) kvalues_iq4nl[nibble]; a sub-block's 16 bytes hold elements 0..15 in their
        // low halves and 16..31 in their high halves.  A fragment holds (ls - 32) kvalue, at most
        // 4064 in magnitude (rounded to fp16 only beyond 2048); d multiplies the MFMA result.
        const uint32_t sb = row + (sl >> 2) * 136;
        const int q = sl & 3;
        uint32_t hdr[2], qs[8];
        lds_read_x1(sb, hdr);
        lds_read_x1(sb + 8 + q * 32, qs);
        lds_landed(hdr);
        lds_landed(qs);
        tail.d = jl_half_bits_to_float(hdr[0]);
        tail.dmin = 0.f;
        const uint32_t scales_h = hdr[0] >> 16, scales_l = hdr[1];
        const h2 bias = {(_Float16)1152.f, (_Float16)1152.f};   // the table bytes with 128 added, under 1024
#pragma unroll
        for (int sub = 0; sub < 2; sub++) {
            const int g = 2 * q + sub;
            const int ls = (int)(((scales_l >> (4 * g)) & 0xFu) | (((scales_h >> (2 * g)) & 3u) << 4)) - 32;
            const _Float16 lsf = (_Float16)(float)ls;
            const h2 ls2 = {lsf, lsf};
            uint32_t lo[4], hi[4];
#pragma unroll
            for (int j = 0; j < 4; j++) {
                lo[j] = jl_iq4nl_lookup4(qs[4 * sub + j] & 0x0F0F0F0Fu) ^ 0x80808080u;
                hi[j] = jl_iq4nl_lookup4((qs[4 * sub + j] >> 4) & 0x0F0F0F0Fu) ^ 0x80808080u;
            }
#pragma unroll
            for (int i = 0; i < 2; i++) {
                f[4 * sub + i] = frag_scaled(lo[2 * i], lo[2 * i + 1], bias, ls2);
                f[4 * sub + 2 + i] = frag_scaled(hi[2 * i], hi[2 * i + 1], bias, ls2);
            }
        }
    } else {
        static_assert(TYPE == JL_Q4_K, "no slice decoder for this type");
        // a quarter of a super-block: 32 nibble bytes; low nibbles are sub-block 2 pair (columns
        // 0..31 of the slice), high nibbles sub-block 2 pair + 1; w = d (sc q) - dmin m
        uint4 h, q0, q1;
        const uint32_t sb = row + (sl >> 2) * 144;
        const int pair = sl & 3;
        lds_read_q4k(sb, sb + 16 + pair * 32, h, q0, q1);
        h2 s0, s1;
        k_scales(h, pair, s0, s1, tail);
        const h2 o0 = s0 * h2{(_Float16)-1024.f, (_Float16)-1024.f};   // exact: at most 63 * 1024
        // the high nibbles stay where they are: a byte 16 q is 1024 + 16 q, times sc / 16 (exact)
        const h2 s1x = s1 * h2{(_Float16)0.0625f, (_Float16)0.0625f};
        const h2 o1 = s1 * h2{(_Float16)-64.f, (_Float16)-64.f};
        const uint32_t qs[8] = {q0.x, q0.y, q0.z, q0.w, q1.x, q1.y, q1.z, q1.w};
#pragma unroll
        for (int i = 0; i < 4; i++) {
            f[i] = frag_times(qs[2 * i] & 0x0F0F0F0Fu, qs[2 * i + 1] & 0x0F0F0F0Fu, s0, o0);
            f[4 + i] = frag_times(qs[2 * i] & 0xF0F0F0F0u, qs[2 * i + 1] & 0xF0F0F0F0u, s1x, o1);
        }
    }
}

// ---- the prologue's arithmetic, by hand.  Written with fmaxf / casts the compiler spends an
// instruction on every |x| and on every operand of a maximum (it must quiet signalling NaNs), four
// on a DPP step and seven on rounding four products to fp16; these are the instructions themselves.

// max(|a|, |b|, |c|, |d|)
__device__ __forceinline__ float max_abs4(const float4 &v) {
    float m;
    asm("v_max3_f32 %0, |%1|, |%2|, |%3|\n\tv_max_f32 %0, %0, |%4|" : "=&v"(m) : "v"(v.x), "v"(v.y), "v"(v.z), "v"(v.w));
    return m;
}
__device__ __forceinline__ float max_raw(float a, float b) {
    float m;
    asm("v_max_f32 %0, %1, %2" : "=v"(m) : "v"(a), "v"(b));
    return m;
}
// max(v, v rotated by N lanes within its row of 16); two wait states between a vector write and a
// DPP read of the same register
#define JL_MAX_ROR(v, N) asm("s_nop 1\n\tv_max_f32_dpp %0, %0, %0 row_ror:" #N " row_mask:0xf bank_mask:0xf" : "+v"(v))
// fp16(a * scale) | fp16(b * scale) << 16, each product rounded once (the scale is a power of two)
__device__ __forceinline__ uint32_t scaled_pair_f16(float a, float b, float scale) {
    uint32_t r;
    asm("v_fma_mixlo_f16 %0, %1, %3, 0\n\tv_fma_mixhi_f16 %0, %2, %3, 0" : "=&v"(r) : "v"(a), "v"(b), "s"(scale));
    return r;
}

__device__ __forceinline__ float skinny_swiglu(float g, float u) { return g * __builtin_amdgcn_rcpf(1.0f + __expf(-g)) * u; }

// Workgroup = 16 Ss compute threads (Ss / 4 waves) + kDmaWaves waves that do nothing but copy tiles.
// An LDS-DMA load holds its wave at issue while the memory system is busy; issued from the compute
// waves that time adds to the arithmetic instead of hiding behind it, so the copies have waves of
// their own and the two kinds meet at one barrier per tile.
constexpr int kDmaWaves = 2;
// ... and so has the fold of the compute waves' partial sums with the epilogue: a chain of LDS
// round trips, exponentials and stores that would otherwise stall the decode of the next tile
// (two waves: one per row block).
constexpr int kFoldWaves = 2;
// buffers of partial sums that a workgroup cycles through, one per group in flight
constexpr int kParities = 3;
constexpr int max_slices(int) { return 32; }
// The prologue's staging area of a compute wave: 8 activation rows x 256 columns as fp16, rows 16
// bytes apart from a multiple of 256 so that the fragment reads of 16 lanes hit all banks.
constexpr int kScratchRow = 528, kScratchPerWave = 8 * kScratchRow;

// 16-byte loads per DMA wave and tile (upper bound): a tile row takes span_bytes + 16 bytes of LDS
// (the padding spreads the 16 rows a wave reads at once over all banks), 16 rows, 128 lanes.
constexpr int loads_per_wave(int type) { return (kGroup * (8 * quad_bytes(type) / 16 + 1) + 64 * kDmaWaves - 1) / (64 * kDmaWaves); }
template <int TYPE> struct Loads { static constexpr int kPerWave = loads_per_wave(TYPE); };
static_assert(Loads<JL_Q8_0>::kPerWave == 18 && Loads<JL_Q4_K>::kPerWave == 10 && Loads<JL_Q6_K>::kPerWave == 14, "");

// ZIN: spans of a row that one workgroup walks itself, one tile after the other, adding their
// results in registers (it then holds ZIN sets of activation fragments); p.Z spans of ZIN each.
// HALF: at most 8 activation rows -- the prologue reads, scales and converts rows 0..7 only (rows
// 8..15 of the row block are zeros either way).
// XH: the activations are binary16 (and a gate/up call may leave binary16).  An instance of its
// own: as a run-time choice inside the prologue it cost the fp32 form 2.5 us per call.
template <int TYPE, int NBB, bool DUAL, int ZIN, bool HALF = false, bool XH = false>
__global__ void __launch_bounds__(512 + 64 * (kDmaWaves + kFoldWaves)) jl_gemm_skinny(SkinnyParams p) {
    static_assert(!HALF || NBB == 1, "a row block of at most 8 rows is the only one");
    constexpr int XR = HALF ? 8 : 16;   // activation rows of a row block the prologue reads
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    constexpr int LD = Loads<TYPE>::kPerWave;
    const int tid = threadIdx.x;
    const int waves = (blockDim.x >> 6) - kDmaWaves - kFoldWaves;   // compute waves
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int lane = tid & 63;
    const int z = blockIdx.x % p.Z;            // this workgroup's run of ZIN spans
    const int row0 = blockIdx.y * (16 * NBB);  // first activation row of this workgroup's row block
    const int lds_row = p.span_bytes + 16;
    const int slots_per_row = lds_row >> 4;
    const int n_loads = (kGroup * slots_per_row + 64 * kDmaWaves - 1) / (64 * kDmaWaves);
    const int stage_bytes = n_loads * 64 * kDmaWaves * 16;
    const int partial_bytes = waves * NBB * 1024;  // one buffer of kParities
    const int total_groups = p.seg_group_begin[p.nseg];
    const int out_rows = DUAL ? kGroup / 2 : kGroup;   // outputs per group

    // LDS: the tile ring, then the partial sums (kParities buffers)
    const uint32_t lds0 = (uint32_t)(uintptr_t)(lvoid *)lds;
    const uint32_t ring0 = lds0;
    uint8_t *ring = lds;
    const uint32_t part0 = lds0 + p.stages * stage_bytes;

    // The weight a row group belongs to.  The table is walked with constant indices: it then stays in
    // scalar registers, where an index computed at run time would turn every use into a load from
    // the argument buffer -- and a load's wait drains the whole tile ring.
    struct Segment {
        const uint8_t *w;
        int rows, group_begin, col_begin;
    };
    auto segment_of = [&](int group) {
        Segment sg = {p.w[0], p.seg_rows[0], 0, 0};
#pragma unroll
        for (int i = 1; i < kMaxSeg; i++) {
            if (i < p.nseg && group >= p.seg_group_begin[i]) {
                sg.w = p.w[i];
                sg.rows = p.seg_rows[i];
                sg.group_begin = p.seg_group_begin[i];
                sg.col_begin = p.seg_col_begin[i];
            }
        }
        return sg;
    };

    // my groups: wg, wg + stride, ... (workgroups of one span share a stride)
    const int wg = blockIdx.x / p.Z;
    const int stride = gridDim.x / p.Z;
    int mine = wg < total_groups ? (total_groups - wg + stride - 1) / stride : 0;

    // Where lane `o` of a fold keeps the four partial sums of (span run zz, row block b, group).
    auto plane_at = [&](int zz, int b, int group, int o) {
        const int64_t slot = (((int64_t)zz * p.row_blocks + blockIdx.y) * NBB + b) * total_groups + group;
        return (floatx4 *)p.planes + slot * 64 + o;
    };
    // The epilogue of one group and row block, by the 64 lanes that hold its sums: lane o has weight
    // row o % 16 of the group against activation rows 16 b + 4 (o / 16) .. + 3 (in a gate/up group
    // the lanes of weight rows 8..15 hold the up rows of outputs 0..7 and store nothing).
    auto finish = [&](int group, int b, int o, const floatx4 &sum, const floatx4 &sum_up) {
        const int n = o & 15, go = o >> 4;
        const Segment sg = segment_of(group);
        const int local = (group - sg.group_begin) * out_rows + n;   // output column inside the weight
        const int m0 = row0 + 16 * b + 4 * go;                       // first of this lane's four activation rows
        if ((DUAL && n >= 8) || local >= sg.rows) return;
        const int64_t at = (int64_t)m0 * p.ldo + p.col_offset + sg.col_begin + local;
        float *dst = p.C + at;
#pragma unroll
        for (int e = 0; e < 4; e++) {
            if (m0 + e >= p.rows) break;
            const float r = DUAL ? skinny_swiglu(sum[e], sum_up[e]) : sum[e];
            if (XH && DUAL && p.c_f16) ((_Float16 *)p.C)[at + e * p.ldo] = (_Float16)r;   // rounded once from the fp32 value
            else if (p.epilogue == JL_RESIDUAL) unsafeAtomicAdd(dst + e * p.ldo, r);   // one add per element, no load to wait for
            else dst[e * p.ldo] = r;
        }
    };

    if (wave >= waves && wave < waves + kDmaWaves) {
        // ---- copy waves.  Slot s of a tile is 16 bytes at LDS offset 16 s: row s / slots_per_row,
        // byte 16 (s % slots_per_row) of the row's span.  A slot past the data (the padding behind
        // each row, slots behind the last row) re-reads a neighbouring real slot -- never one
        // shared address, which every compute unit would then hammer.
        const int dw = wave - waves;
        const int span_slots = p.span_bytes >> 4;
        // the few instructions these waves issue go first: the copy is what everything waits for
        __builtin_amdgcn_s_setprio(3);
        // What a lane adds to the tile's first byte never changes: its row's offset, its place in
        // the span and, for the up half of a gate/up group, the distance between the two weights
        // (a gate/up call has one segment).  An issue is then one 64-bit add and the load.
        int slot_in[LD], slot_wrow[LD];
        int64_t slot_off[LD], slot_off_row0[LD];
        // slot (j kDmaWaves + dw) 64 + lane: one division for j = 0, then steps of 64 kDmaWaves slots
        const int step_rows = (64 * kDmaWaves) / slots_per_row, step_within = (64 * kDmaWaves) % slots_per_row;
        int srow = (dw * 64 + lane) / slots_per_row;
        int swithin = dw * 64 + lane - srow * slots_per_row;
        const int64_t up_distance = DUAL ? (int64_t)(p.w_up - p.w[0]) : 0;
#pragma unroll
        for (int j = 0; j < LD; j++) {
            const int row = srow < kGroup ? srow : kGroup - 1;
            const int within = swithin < span_slots ? swithin : span_slots - 1;
            slot_wrow[j] = DUAL ? (row & 7) : row;
            slot_in[j] = z * ZIN * p.span_bytes + within * 16;
            const int64_t up = (DUAL && row >= 8) ? up_distance : 0;
            slot_off_row0[j] = up + slot_in[j];
            slot_off[j] = slot_off_row0[j] + (int64_t)(slot_wrow[j] * p.row_bytes);
            srow += step_rows;
            swithin += step_within;
            if (swithin >= slots_per_row) {
                swithin -= slots_per_row;
                srow++;
            }
        }
        // tile t = span t % ZIN of group wg + (t / ZIN) stride
        auto issue = [&](int t, int st) {
            const int group = wg + (t / ZIN) * stride;
            const int span_off = (t % ZIN) * p.span_bytes;
            const Segment sg = segment_of(group);
            const int first_row = (group - sg.group_begin) * out_rows;
            const int64_t base_off = (int64_t)first_row * p.row_bytes + span_off;
            const uint8_t *w_gate = sg.w + base_off;
            asm volatile("" : "+s"(w_gate));   // in scalar registers before any per-lane arithmetic
            uint8_t *dst = ring + st * stage_bytes;
            if (first_row + out_rows <= sg.rows && p.row_blocks == 1) {
                // every row of the group exists (uniform; all groups but a weight's last), and
                // nobody else reads this tile: read once, marked so
#pragma unroll
                for (int j = 0; j < LD; j++) {
                    if (j >= n_loads) break;
                    __builtin_amdgcn_global_load_lds((gvoid *)(w_gate + slot_off[j]),
                                                     (lvoid *)(dst + (j * kDmaWaves + dw) * 1024), 16, 0, kStreamNonTemporal);
                }
            } else if (first_row + out_rows <= sg.rows) {
                // the other row blocks' workgroups read the same tile from the same L2: default policy
#pragma unroll
                for (int j = 0; j < LD; j++) {
                    if (j >= n_loads) break;
                    __builtin_amdgcn_global_load_lds((gvoid *)(w_gate + slot_off[j]),
                                                     (lvoid *)(dst + (j * kDmaWaves + dw) * 1024), 16, 0, 0);
                }
            } else {
#pragma unroll
                for (int j = 0; j < LD; j++) {
                    if (j >= n_loads) break;
                    // past the weight's last row: re-read the group's first row
                    const int wrow = first_row + slot_wrow[j] >= sg.rows ? 0 : slot_wrow[j];
                    __builtin_amdgcn_global_load_lds((gvoid *)(w_gate + slot_off_row0[j] + (int64_t)wrow * p.row_bytes),
                                                     (lvoid *)(dst + (j * kDmaWaves + dw) * 1024), 16, 0, 0);
                }
            }
        };
        const int tiles = mine * ZIN;
        int issued = 0, next_stage = 0;
        for (; issued < p.stages - 1 && issued < tiles; issued++) {
            issue(issued, next_stage);
            next_stage = next_stage + 1 == p.stages ? 0 : next_stage + 1;
        }
        for (int t = 0; t < tiles; t++) {
            // tiles issued after tile t may stay in flight
            wait_vm((issued - t - 1) * n_loads);
            __builtin_amdgcn_s_barrier();
            // the stage of tile t - 1 is free now: every compute wave is past its reads
            if (issued < tiles) {
                issue(issued, next_stage);
                next_stage = next_stage + 1 == p.stages ? 0 : next_stage + 1;
                issued++;
            }
        }
        if (mine > 0) __builtin_amdgcn_s_barrier();
    } else if (wave >= waves + kDmaWaves) {
        // ---- fold waves.  The partial sums of group it (buffer it % kParities) are complete one
        // tile after the group's last one -- the late compute waves multiply a tile behind -- and
        // are overwritten three groups later, behind barriers these waves take part in.  With two
        // row blocks each fold wave takes one (a fold of both took longer than a tile when the
        // workgroup walks a single span), else the first does the work.  A partial is what one lane of one
        // compute wave held: weight row o % 16 of the group against activation rows
        // 16 b + 4 (o / 16) .. + 3, for lane o and row block b; in a gate/up group weight rows 8..15
        // are the up rows of outputs 0..7.  Lane o of this wave adds the waves' partials of its
        // (b, o) in wave order and applies the epilogue.
        const int o = lane;
        // with two fold waves and two row blocks each takes one block (the fold of a group has one
        // tile's time when the workgroup walks a single span)
        const int fw = wave - waves - kDmaWaves;
        // its few instructions go ahead of the compute waves' on the SIMD they share: every
        // barrier between two folds waits for this wave
        __builtin_amdgcn_s_setprio(2);
        auto fold = [&](int group, int par) {
            const uint32_t pbase = part0 + par * partial_bytes + o * 16;
#pragma unroll
            for (int b = 0; b < NBB; b++) {
                if (kFoldWaves > 1 && (NBB > 1 ? b != fw : fw != 0)) continue;
                // all of the (at most eight) compute waves' partials in one round trip
                floatx4 v[8], u[8];
#pragma unroll
                for (int j = 0; j < 8; j++) {
                    const uint32_t a = pbase + (j < waves ? j : 0) * (NBB * 1024) + b * 1024;
                    asm volatile("ds_read_b128 %0, %1" : "=&v"(v[j]) : "v"(a) : "memory");
                    // (lanes 56..63 read past their own row block here; in range, and unused)
                    if constexpr (DUAL) asm volatile("ds_read_b128 %0, %1 offset:128" : "=&v"(u[j]) : "v"(a) : "memory");
                }
                asm volatile("s_waitcnt lgkmcnt(0)"
                             : "+v"(v[0]), "+v"(v[1]), "+v"(v[2]), "+v"(v[3]), "+v"(v[4]), "+v"(v[5]), "+v"(v[6]), "+v"(v[7])
                             : : "memory");
                if constexpr (DUAL)
                    asm volatile("" : "+v"(u[0]), "+v"(u[1]), "+v"(u[2]), "+v"(u[3]), "+v"(u[4]), "+v"(u[5]), "+v"(u[6]), "+v"(u[7]));
                floatx4 sum = v[0], sum_up = u[0];
#pragma unroll
                for (int j = 1; j < 8; j++) {
                    if (j < waves) {
                        sum += v[j];
                        if constexpr (DUAL) sum_up += u[j];
                    }
                }
                if (p.Z > 1) {
                    // this span's partial sums, 16 bytes per lane: the workgroup that arrives last
                    // adds the spans' in span order (the tail of the kernel)
                    asm volatile("" : "+v"(sum));   // (plain vector arithmetic has run on it: no matrix-pipe hazard)
                    agent_store_f4(plane_at(z, b, group, o), sum);
                    continue;
                }
                finish(group, b, o, sum, sum_up);
            }
        };
        // The late compute waves (below) finish group it during the tile after its last one, so
        // its partial sums are complete at the barrier of tile (it + 1) ZIN + 1; they sit in buffer
        // it % 3, which the early waves write again at the end of group it + 3.
        const int tiles = mine * ZIN;
        int folded = 0;
        for (int t = 0; t < tiles; t++) {
            __builtin_amdgcn_s_barrier();
            if (folded < mine && (folded + 1) * ZIN + 1 <= t) {
                fold(wg + folded * stride, folded % kParities);
                folded++;
            }
        }
        if (mine > 0) {
            __builtin_amdgcn_s_barrier();
            for (; folded < mine; folded++) fold(wg + folded * stride, folded % kParities);
        }
        __builtin_amdgcn_s_setprio(0);
    } else {
    // ---- compute waves
    const int c = lane & 15;                   // weight row of the group; activation row of a row block
    const int g = lane >> 4;                   // which of the wave's four slices
    const int sl = 4 * wave + g;               // slice inside the span

    // Activation fragments: 64 consecutive columns of NBB x 16 rows, kept for the whole kernel.
    // Read as fp32 (while the first tiles are on their way) and rounded to fp16 behind a
    // power-of-two scale per row and wave: the largest magnitude of the row's 256 columns this wave
    // multiplies is brought into [2^9, 2^10), which keeps huge rows finite, tiny rows out of
    // fp16's subnormals and the sum of a sub-block's 32 activations inside fp16's range.  The
    // results of activation row r sit in lane group r / 4 of every weight row's lanes, so each lane
    // fetches the four scales it has to undo from the lanes that computed them.
    half8 af[NBB][ZIN][8];
    half8 sums[NBB][ZIN];     // Q4_K: the two sub-blocks' activation sums, each as hi + lo, as k slots
    floatx4 undo[NBB][ZIN];
    {
        // Every load of the prologue is issued before the first value is used, and every load
        // instruction reads one row's 1 KB run of the wave's 256 columns: lane l holds columns
        // 4 l .. 4 l + 3 of row r in register r.  (Loads shaped like the fragments -- a lane
        // fetching pieces of its own row and slice -- touch 16 rows per instruction and took
        // 2 us longer per launch: the cache looks up one line per clock.)  The rows are scaled,
        // rounded to fp16 and turned into fragments through LDS, eight rows at a time, in a
        // region of the wave's own: the last ring stage and the partial sums behind it, neither of
        // which anybody touches before the first tile has been multiplied.
        uint8_t *scr = lds + (p.stages - 1) * stage_bytes + wave * kScratchPerWave;
        float4 x[NBB * ZIN][XR];
#pragma unroll
        for (int b = 0; b < NBB; b++) {
#pragma unroll
            for (int q = 0; q < ZIN; q++) {
                const int col = 64 * ((z * ZIN + q) * p.Ss + 4 * wave) + 4 * lane;
                // rows past the last active one re-read it (their results are never stored): no
                // branch and no zero fill per row, and the address moves by one row length
                const int first = row0 + 16 * b;
                const int64_t begin = (int64_t)(first < p.rows ? first : p.rows - 1) * p.k + col;
                if constexpr (XH) {
                    // binary16 activations: the lane's four values arrive as two dwords and are
                    // widened below, once every load has been issued
                    const _Float16 *rowp = (const _Float16 *)p.X + begin;
#pragma unroll
                    for (int r = 0; r < XR; r++) {
                        const uint2 h = *(const uint2 *)rowp;
                        x[b * ZIN + q][r] = float4{__uint_as_float(h.x), __uint_as_float(h.y), 0.f, 0.f};
                        if (first + r + 1 < p.rows) rowp += p.k;
                    }
                } else {
                    const float *rowp = p.X + begin;
#pragma unroll
                    for (int r = 0; r < XR; r++) {
                        x[b * ZIN + q][r] = *(const float4 *)rowp;
                        if (first + r + 1 < p.rows) rowp += p.k;
                    }
                }
            }
        }
        if constexpr (XH) {
#pragma unroll
            for (int i = 0; i < NBB * ZIN; i++) {
#pragma unroll
                for (int r = 0; r < XR; r++) {
                    const h2 lo = __builtin_bit_cast(h2, __float_as_uint(x[i][r].x));
                    const h2 hi = __builtin_bit_cast(h2, __float_as_uint(x[i][r].y));
                    x[i][r] = float4{(float)lo[0], (float)lo[1], (float)hi[0], (float)hi[1]};
                }
            }
        }
#pragma unroll
        for (int b = 0; b < NBB; b++) {
#pragma unroll
            for (int q = 0; q < ZIN; q++) {
                const float4 (&xs)[XR] = x[b * ZIN + q];
                // The largest magnitude of each row's 256 columns.  Sixteen registers of per-lane
                // maxima are folded over the lanes and halved twice on the way (a swap of lane
                // halves puts row r and row r + 8 side by side, a swap of lane quarters rows r and
                // r + 4), so lane group g ends with the maxima of rows 4 g .. 4 g + 3 -- the rows
                // whose results its lanes will hold.
                float v16[16];
#pragma unroll
                for (int r = 0; r < 16; r++) v16[r] = r < XR ? max_abs4(xs[r]) : 0.f;
                float v8[8], v4[4];
#pragma unroll
                for (int r = 0; r < 8; r++) {
                    const auto sw = __builtin_amdgcn_permlane32_swap(__float_as_uint(v16[r]), __float_as_uint(v16[r + 8]), false, false);
                    v8[r] = max_raw(__uint_as_float(sw[0]), __uint_as_float(sw[1]));
                }
#pragma unroll
                for (int r = 0; r < 4; r++) {
                    const auto sw = __builtin_amdgcn_permlane16_swap(__float_as_uint(v8[r]), __float_as_uint(v8[r + 4]), false, false);
                    v4[r] = max_raw(__uint_as_float(sw[0]), __uint_as_float(sw[1]));
                }
                // rotations within the 16 lanes: every lane ends with the maximum
#pragma unroll
                for (int j = 0; j < 4; j++) {
                    JL_MAX_ROR(v4[j], 8);
                    JL_MAX_ROR(v4[j], 4);
                    JL_MAX_ROR(v4[j], 2);
                    JL_MAX_ROR(v4[j], 1);
                }
                // amax = 1.f * 2^(E - 127): multiply by 2^(136 - E), undo with 2^(E - 136); the
                // row's largest value lands in [2^9, 2^10), which keeps huge rows finite, tiny rows
                // out of fp16's subnormals and a sub-block's sum of 32 inside fp16's range
                uint32_t inv4[4];
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    int E = (int)((__float_as_uint(v4[e]) >> 23) & 0xFF);
                    E = E < 12 ? 12 : E;
                    undo[b][q][e] = __uint_as_float((uint32_t)(E - 9) << 23);
                    inv4[e] = (uint32_t)(263 - E) << 23;
                }
                // (the scale of row r, a scalar operand of its conversions: lane group r / 4 holds it)
                float inv[XR];
#pragma unroll
                for (int r = 0; r < XR; r++) inv[r] = __uint_as_float(__builtin_amdgcn_readlane(inv4[r & 3], 16 * (r >> 2)));
                if constexpr (HALF) {
                    const _Float16 z16 = (_Float16)0.f;
#pragma unroll
                    for (int i = 0; i < 8; i++) af[b][q][i] = half8{z16, z16, z16, z16, z16, z16, z16, z16};
                }
#pragma unroll
                for (int pass = 0; pass < XR / 8; pass++) {
#pragma unroll
                    for (int rr = 0; rr < 8; rr++) {
                        const int r = 8 * pass + rr;
                        *(uint2 *)(scr + rr * kScratchRow + lane * 8) =
                            uint2{scaled_pair_f16(xs[r].x, xs[r].y, inv[r]), scaled_pair_f16(xs[r].z, xs[r].w, inv[r])};
                    }
                    __builtin_amdgcn_wave_barrier();   // (LDS serves a wave's accesses in order)
                    if ((c >> 3) == pass) {
#pragma unroll
                        for (int i = 0; i < 8; i++) af[b][q][i] = *(const half8 *)(scr + (c & 7) * kScratchRow + 128 * g + 16 * i);
                    }
                    __builtin_amdgcn_wave_barrier();
                }
                if constexpr (kHasMins<TYPE>) {
                    // sums of the values the MFMAs will see: at most 32 x 2^10, exact in fp32
                    float part[2] = {0.f, 0.f};
                    const h2 ones = {(_Float16)1.f, (_Float16)1.f};
#pragma unroll
                    for (int i = 0; i < 8; i++) {
                        const half8 h = af[b][q][i];
#pragma unroll
                        for (int e = 0; e < 8; e += 2)
                            part[i >> 2] = __builtin_amdgcn_fdot2(h2{h[e], h[e + 1]}, ones, part[i >> 2], false);
                    }
                    const _Float16 z16 = (_Float16)0.f;
                    const _Float16 h0 = (_Float16)part[0], h1 = (_Float16)part[1];
                    sums[b][q] = half8{h0, (_Float16)(part[0] - (float)h0), h1, (_Float16)(part[1] - (float)h1), z16, z16, z16, z16};
                }
            }
        }
    }
    // One tile: the slice's fragments against the activation fragments of span q, added to `total`.
    auto multiply = [&](int q, const half8 (&wf)[8], const Q4KTail &tail, floatx4 (&total)[NBB]) {
#pragma unroll
        for (int b = 0; b < NBB; b++) {
            floatx4 acc0 = {0.f, 0.f, 0.f, 0.f}, acc1 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int i = 0; i < 8; i += 2) {
                acc0 = __builtin_amdgcn_mfma_f32_16x16x32_f16(af[b][q][i], wf[i], acc0, 0, 0, 0);
                acc1 = __builtin_amdgcn_mfma_f32_16x16x32_f16(af[b][q][i + 1], wf[i + 1], acc1, 0, 0, 0);
            }
            if constexpr (kHasMins<TYPE>) {
                const floatx4 zero = {0.f, 0.f, 0.f, 0.f};
                const floatx4 accm = __builtin_amdgcn_mfma_f32_16x16x32_f16(sums[b][q], tail.mins, zero, 0, 0, 0);
                total[b] += ((acc0 + acc1) * tail.d - accm * tail.dmin) * undo[b][q];
            } else if constexpr (kPostScale<TYPE>) {
                total[b] += (acc0 + acc1) * (tail.d * undo[b][q]);
            } else {
                total[b] += (acc0 + acc1) * undo[b][q];
            }
        }
    };
    // plain arithmetic happened on the MFMA results: the compiler placed the wait states itself
    auto publish = [&](int it, floatx4 (&total)[NBB]) {
        asm volatile("" : "+v"(total[0]));
        const uint32_t pw = part0 + (it % kParities) * partial_bytes + wave * (NBB * 1024) + lane * 16;
#pragma unroll
        for (int b = 0; b < NBB; b++) lds_write_f4(pw + b * 1024, total[b]);
    };
    // The two compute waves of a SIMD (w and w + 4) run half a tile apart, so that one of them
    // decodes (vector ALU) while the other multiplies (matrix pipe): after the barrier of tile t
    // the early wave decodes tile t and multiplies it; the late wave first multiplies tile t - 1,
    // whose fragments it holds, and then decodes tile t.  In lock step both decoded first and the
    // second one's MFMAs, a chain of dependent accumulations, ended the tile alone.
    if (wave < 4) {
        for (int it = 0; it < mine; it++) {
            floatx4 total[NBB];
#pragma unroll
            for (int b = 0; b < NBB; b++) total[b] = floatx4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int q = 0; q < ZIN; q++) {
                const int t = it * ZIN + q;
                __builtin_amdgcn_s_barrier();   // tile t has landed
                half8 wf[8];
                Q4KTail tail;
                decode_slice<TYPE>(ring0 + (t % p.stages) * stage_bytes + c * lds_row, sl, wf, tail);
                asm volatile("" : "+v"(wf[0]), "+v"(wf[7]));
                multiply(q, wf, tail, total);
            }
            publish(it, total);
        }
    } else {
        half8 wf[8];
        Q4KTail tail;
        floatx4 total[NBB];
#pragma unroll
        for (int b = 0; b < NBB; b++) total[b] = floatx4{0.f, 0.f, 0.f, 0.f};
        for (int it = 0; it < mine; it++) {
#pragma unroll
            for (int q = 0; q < ZIN; q++) {
                const int t = it * ZIN + q;
                __builtin_amdgcn_s_barrier();   // tile t has landed
                if (t > 0) {
                    // tile t - 1: span (q - 1) mod ZIN, the last of its group when q == 0
                    multiply(q == 0 ? ZIN - 1 : q - 1, wf, tail, total);
                    if (q == 0) {
                        publish(it - 1, total);
#pragma unroll
                        for (int b = 0; b < NBB; b++) total[b] = floatx4{0.f, 0.f, 0.f, 0.f};
                    }
                }
                decode_slice<TYPE>(ring0 + (t % p.stages) * stage_bytes + c * lds_row, sl, wf, tail);
                asm volatile("" : "+v"(wf[0]), "+v"(wf[7]));
            }
        }
        if (mine > 0) {
            multiply(ZIN - 1, wf, tail, total);
            publish(mine - 1, total);
        }
    }
    if (mine > 0) __builtin_amdgcn_s_barrier();
    }

    // ---- rows cut across workgroups (Z > 1): the workgroup of a set that finishes last adds the
    // set's partial sums in span order and applies the epilogue -- no launch behind this one.  The
    // Z workgroups of a set (same groups, one span run each) count themselves in on the set's
    // counter once their partial sums have been written through to device scope; the one that draws
    // the last number reads every span's planes from there (its own included: one order of addition
    // whoever is last) and finishes the set's groups with all twelve waves.  Nobody waits for
    // anybody: a workgroup that is not last is done.  The counter is back at zero for the next call.
    if (p.Z > 1 && mine > 0) {
        vm_drained();   // the fold waves' plane stores have completed
        __builtin_amdgcn_s_barrier();
        uint32_t *flag = (uint32_t *)lds;      // the ring is no longer in use
        if (wave == waves + kDmaWaves && lane == 0) {
            uint32_t *counter = p.arrivals + blockIdx.y * stride + wg;
            const uint32_t before = __hip_atomic_fetch_add(counter, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            if (before == (uint32_t)(p.Z - 1)) __hip_atomic_store(counter, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            *flag = before;
        }
        __builtin_amdgcn_s_barrier();
        if (*flag != (uint32_t)(p.Z - 1)) return;
        // This wave's (group, row block) pairs are wave, wave + 12, ...; a pair has Z planes.  The
        // loads of up to kChunk planes are in flight at a time (one round trip to memory per chunk)
        // and are added in span order; a pair is finished when its last plane has been added.
        const int all_waves = blockDim.x >> 6;
        const int pairs = mine * NBB;
        const int my_pairs = wave < pairs ? (pairs - wave + all_waves - 1) / all_waves : 0;
        const int items = my_pairs * p.Z;
        constexpr int kChunk = DUAL ? 8 : 16;
        floatx4 sum = {0.f, 0.f, 0.f, 0.f}, sum_up = {0.f, 0.f, 0.f, 0.f};
        // (two walks over the same list of (pair, span run): one issues loads, one adds; counters
        // instead of a division per item)
        int lq = wave, lz = 0, aq = wave, az = 0;
        for (int base = 0; base < items; base += kChunk) {
            floatx4 v[kChunk], u[kChunk];
#pragma unroll
            for (int j = 0; j < kChunk; j++) {
                // (slots past the list hold zeros: every register of the chunk is defined when the
                // one wait below takes them all)
                v[j] = floatx4{0.f, 0.f, 0.f, 0.f};
                u[j] = floatx4{0.f, 0.f, 0.f, 0.f};
                if (base + j < items) {
                    const int group = wg + (lq / NBB) * stride, b = lq % NBB;
                    v[j] = agent_load_f4(plane_at(lz, b, group, lane));
                    // (a gate/up group keeps the up rows' sums eight lanes on; lanes that have no
                    // such neighbour read their own group's first lanes and drop the result)
                    if constexpr (DUAL) u[j] = agent_load_f4(plane_at(lz, b, group, (lane + 8) & 63));
                    if (++lz == p.Z) {
                        lz = 0;
                        lq += all_waves;
                    }
                }
            }
            // one wait for the chunk; every destination passes through it, so that no use of one
            // can move ahead of it
            if constexpr (DUAL) {
                asm volatile("s_waitcnt vmcnt(0)"
                             : "+v"(v[0]), "+v"(v[1]), "+v"(v[2]), "+v"(v[3]), "+v"(v[4]), "+v"(v[5]), "+v"(v[6]), "+v"(v[7]),
                               "+v"(u[0]), "+v"(u[1]), "+v"(u[2]), "+v"(u[3]), "+v"(u[4]), "+v"(u[5]), "+v"(u[6]), "+v"(u[7])
                             : : "memory");
            } else {
                asm volatile("s_waitcnt vmcnt(0)"
                             : "+v"(v[0]), "+v"(v[1]), "+v"(v[2]), "+v"(v[3]), "+v"(v[4]), "+v"(v[5]), "+v"(v[6]), "+v"(v[7]),
                               "+v"(v[8]), "+v"(v[9]), "+v"(v[10]), "+v"(v[11]), "+v"(v[12]), "+v"(v[13]), "+v"(v[14]), "+v"(v[15])
                             : : "memory");
            }
#pragma unroll
            for (int j = 0; j < kChunk; j++) {
                if (base + j < items) {
                    sum += v[j];
                    if constexpr (DUAL) sum_up += u[j];
                    if (++az == p.Z) {
                        finish(wg + (aq / NBB) * stride, aq % NBB, lane, sum, sum_up);
                        sum = floatx4{0.f, 0.f, 0.f, 0.f};
                        sum_up = floatx4{0.f, 0.f, 0.f, 0.f};
                        az = 0;
                        aq += all_waves;
                    }
                }
            }
        }
    }
}

// Workgroups per span: one workgroup per compute unit and span (the ring takes most of the LDS),
// fewer for less work.  The row blocks of a call share the chip: workgroup (x, y) runs beside
// (x, y + 1), and with a grid width that is a multiple of 8 both land on the same XCD, whose L2
// then serves the later readers of every tile -- unless rounding down to that multiple would idle
// more than a fifth of the chip (Q4_K down projection of 12288 columns at 96 rows: 8 instead of 14
// workgroups per span took 46 us instead of 34).
int workgroups_per_span(int compute_units, int row_blocks, int Z, int groups) {
    int per_span = compute_units / row_blocks / Z;
    if (row_blocks > 1 && per_span / 8 * 8 * 5 >= per_span * 4) per_span = per_span / 8 * 8;
    if (per_span < 1) per_span = 1;
    return per_span > groups ? groups : per_span;
}

template <int TYPE, int NBB, bool DUAL, int ZIN, bool HALF, bool XH>
int launch_of(jl_context *ctx, const SkinnyParams &p, int threads, int lds, int groups) {
    auto fn = jl_gemm_skinny<TYPE, NBB, DUAL, ZIN, HALF, XH>;
    static jl_lds_limit_flags configured;
    {
        const int st = jl_raise_lds_limit(configured, ctx->device, (const void *)fn, 160 * 1024);
        if (st != JL_OK) return st;
    }
    const int per_span = workgroups_per_span(ctx->compute_units, p.row_blocks, p.Z, groups);
    if (p.Z > 1 && per_span * p.row_blocks > JL_CONTEXT_ARRIVALS) {
        return jl_fail(JL_ERR_UNSUPPORTED, "jl_gemm: %d workgroup sets exceed the context's %d arrival counters",
                       per_span * p.row_blocks, JL_CONTEXT_ARRIVALS);
    }
    hipLaunchKernelGGL(fn, dim3(per_span * p.Z, p.row_blocks), dim3(threads + 64 * (kDmaWaves + kFoldWaves)), lds,
                       ctx->stream, p);
    JL_HIP(hipGetLastError());
    return JL_OK;
}

template <int TYPE, int NBB, bool DUAL, int ZIN, bool HALF = false>
int launch(jl_context *ctx, const SkinnyParams &p, int threads, int lds, int groups) {
    return launch_of<TYPE, NBB, DUAL, ZIN, HALF, JL_SKINNY_XH>(ctx, p, threads, lds, groups);
}

template <int TYPE, bool DUAL>
int launch_nbb(jl_context *ctx, const SkinnyParams &p, int nbb, int zin, int threads, int lds, int groups) {
    if (nbb == 1 && p.rows <= 8) {
        return zin == 2 ? launch<TYPE, 1, DUAL, 2, true>(ctx, p, threads, lds, groups)
                        : launch<TYPE, 1, DUAL, 1, true>(ctx, p, threads, lds, groups);
    }
    if (nbb == 1) {
        return zin == 2 ? launch<TYPE, 1, DUAL, 2>(ctx, p, threads, lds, groups)
                        : launch<TYPE, 1, DUAL, 1>(ctx, p, threads, lds, groups);
    }
    return launch<TYPE, 2, DUAL, 1>(ctx, p, threads, lds, groups);
}

}  // namespace

// One launch over a window of the weights' columns: `window_slices` 64-column slices from slice
// `first_slice` on (0 slices: the whole row).  The kernel needs nothing for it but bases that start at
// the window -- a weight row's stride and an activation row's stride stay those of the whole row.
// `probe`: says in *taken whether the launch would be made, and makes none.
static int skinny_window(jl_context *ctx, const jl_weight *const *weights, int count, const float *X,
                         const _Float16 *X16, float *C, bool c_f16, int rows, int64_t ldo, int64_t col_offset,
                         int epilogue, float *planes, size_t plane_bytes, double other_us, bool *taken,
                         int first_slice, int window_slices, bool probe) {
    *taken = false;
    const int type = weights[0]->type;
    const int k = (int)weights[0]->cols;
    const bool dual = epilogue == JL_SWIGLU;
    if (rows >= 512 || k % 256 != 0 || count > kMaxSeg) return JL_OK;
    const int S = window_slices ? window_slices : k / 64;
    const int row_blocks = (rows + 31) / 32;
    const int nbb = jl_skinny_padded_rows(rows) / 16;
    const int quad = quad_bytes(type);
    if (quad == 0) return JL_OK;
    for (int i = 0; i < count; i++)
        if (weights[i]->type != type) return JL_OK;
    // a span is a whole number of 256-column blocks and of 16-byte pieces (Q6_K: 8 blocks of 210
    // bytes, IQ4_XS: 2 of 136), and so is a row
    int Ss = max_slices(nbb);
    while (Ss > 4 && (S % Ss || (Ss / 4 * quad) % 16)) Ss -= 4;
    if (S % Ss || (Ss / 4 * quad) % 16 || (k / 256 * quad) % 16 || (first_slice / 4 * quad) % 16) return JL_OK;
    // up to 16 rows: a workgroup walks two spans itself (no partial sums to fold for rows of up to
    // 4096 columns); more rows leave no registers for a second set of activation fragments
    const int zin = (nbb == 1 && (S / Ss) % 2 == 0) ? 2 : 1;
    const int Z = S / Ss / zin;

    if (rows > 64) {
        // 65 .. 511 rows run as three to sixteen row blocks, each streaming the whole weight over its
        // share of the chip: what this costs grows with blocks x weights, and the call is taken when
        // that is less than the caller's estimate for its other way.  Microseconds, fitted to graph
        // replays of the calls of a Llama-3.2-1B layer (Q8_0) and of 8B-shaped layers (Q4_K, Q6_K,
        // Q5_K) at 65 .. 384 rows: 10 + 0.155 x row blocks x million weights / share of the chip in use.
        double millions = 0.0;
        int all_groups = 0;
        for (int i = 0; i < count; i++) millions += (double)weights[i]->rows * (S * 64) * 1e-6;   // (of the window)
        for (int i = 0; i < (dual ? 1 : count); i++) all_groups += ((int)weights[i]->rows + (dual ? 8 : 16) - 1) / (dual ? 8 : 16);
        const int per_span = workgroups_per_span(ctx->compute_units, row_blocks, Z, all_groups);
        double share = (double)per_span * Z * row_blocks / ctx->compute_units;
        if (share > 1.0) share = 1.0;
        if (10.0 + 0.155 * row_blocks * millions / share >= other_us) return JL_OK;
    }

    SkinnyParams p{};
    p.nseg = dual ? 1 : count;
    int groups = 0, col = 0;
    const int per_group = dual ? 8 : 16;
    for (int i = 0; i < p.nseg; i++) {
        p.w[i] = weights[i]->blocks + (int64_t)(first_slice / 4) * quad;
        p.seg_rows[i] = (int)weights[i]->rows;
        p.seg_group_begin[i] = groups;
        p.seg_col_begin[i] = col;
        groups += ((int)weights[i]->rows + per_group - 1) / per_group;
        col += (int)weights[i]->rows;
    }
    p.seg_group_begin[p.nseg] = groups;
    p.w_up = dual ? weights[1]->blocks : nullptr;
    p.X = JL_SKINNY_XH ? (const float *)(X16 + (int64_t)first_slice * 64) : X + (int64_t)first_slice * 64;
    p.C = C;
    p.c_f16 = c_f16 ? 1 : 0;
    p.planes = planes;
    p.arrivals = ctx->arrivals;
    p.rows = rows;
    p.k = k;
    p.ldo = ldo;
    p.col_offset = col_offset;
    p.epilogue = epilogue;
    p.row_bytes = k / jl_block_elems(type) * jl_block_bytes(type);
    p.Ss = Ss;
    p.Z = Z;
    p.row_blocks = row_blocks;
    p.span_bytes = Ss / 4 * quad;
    if (Z > 1 && (size_t)Z * (16 * nbb * row_blocks) * groups * 16 * sizeof(float) > plane_bytes) return JL_OK;

    const int threads = 16 * Ss;   // compute threads; the copy and fold waves come on top
    const int per_wave = loads_per_wave(type);
    const int n_loads = (kGroup * ((p.span_bytes + 16) / 16) + 64 * kDmaWaves - 1) / (64 * kDmaWaves);
    if (n_loads > per_wave) return JL_OK;
    const int stage_bytes = n_loads * 64 * kDmaWaves * 16;
    const int partial = kParities * (threads / 64) * nbb * 1024;
    int stages = (160 * 1024 - partial) / stage_bytes;
    if (stages > 4) stages = 4;
    if (stages < 2) return JL_OK;
    // the prologue's staging area is the last stage and the partial sums behind it
    if ((threads / 64) * kScratchPerWave > stage_bytes + partial) return JL_OK;
    p.stages = stages;
    const int lds = partial + stages * stage_bytes;
    *taken = true;
    if (probe) return JL_OK;

    switch (type) {
        case JL_Q8_0:
            return dual ? launch_nbb<JL_Q8_0, true>(ctx, p, nbb, zin, threads, lds, groups)
                        : launch_nbb<JL_Q8_0, false>(ctx, p, nbb, zin, threads, lds, groups);
        case JL_Q4_0:
            return dual ? launch_nbb<JL_Q4_0, true>(ctx, p, nbb, zin, threads, lds, groups)
                        : launch_nbb<JL_Q4_0, false>(ctx, p, nbb, zin, threads, lds, groups);
        case JL_Q4_K:
            return dual ? launch_nbb<JL_Q4_K, true>(ctx, p, nbb, zin, threads, lds, groups)
                        : launch_nbb<JL_Q4_K, false>(ctx, p, nbb, zin, threads, lds, groups);
        case JL_Q6_K:
            return dual ? launch_nbb<JL_Q6_K, true>(ctx, p, nbb, zin, threads, lds, groups)
                        : launch_nbb<JL_Q6_K, false>(ctx, p, nbb, zin, threads, lds, groups);
        case JL_Q5_K:
            return dual ? launch_nbb<JL_Q5_K, true>(ctx, p, nbb, zin, threads, lds, groups)
                        : launch_nbb<JL_Q5_K, false>(ctx, p, nbb, zin, threads, lds, groups);
        case JL_Q4_1:
            return dual ? launch_nbb<JL_Q4_1, true>(ctx, p, nbb, zin, threads, lds, groups)
                        : launch_nbb<JL_Q4_1, false>(ctx, p, nbb, zin, threads, lds, groups);
        case JL_Q5_0:
            return dual ? launch_nbb<JL_Q5_0, true>(ctx, p, nbb, zin, threads, lds, groups)
                        : launch_nbb<JL_Q5_0, false>(ctx, p, nbb, zin, threads, lds, groups);
        case JL_IQ4_XS:
            return dual ? launch_nbb<JL_IQ4_XS, true>(ctx, p, nbb, zin, threads, lds, groups)
                        : launch_nbb<JL_IQ4_XS, false>(ctx, p, nbb, zin, threads, lds, groups);
        default:
            *taken = false;
            return JL_OK;
    }
}

// Sets *taken to false, launching nothing, when the shape is not one this kernel takes; the caller
// then uses the tiled GEMM.  (JL_SKINNY_XH: X16 is read, else X.)
int JL_SKINNY_ENTRY(jl_context *ctx, const jl_weight *const *weights, int count, const float *X,
                    const _Float16 *X16, float *C, bool c_f16, int rows, int64_t ldo, int64_t col_offset,
                    int epilogue, float *planes, size_t plane_bytes, double other_us, bool *taken) {
    // A row is cut into equal spans of whole 256-column blocks, at most eight blocks each, one compute
    // wave per block: a row of 43 blocks (11 008 columns, the feed-forward width of many 7B models) or
    // of 74 (18 944) has no such cut but spans of one or two blocks, on one or two compute waves (100
    // blocks, 25 600 columns: five).  A plain or residual projection over a row whose
    // widest equal span is under six blocks is two launches instead: the whole eights of its blocks,
    // then the rest as one span that adds to what the first left (measured: 4-14 x at 11 008 columns,
    // 3-5 x at 18 944, 1.4 x at 64 rows of 25 600).
    *taken = false;
    const int k = (int)weights[0]->cols;
    const int blocks = k / 256;
    int widest = 8;
    while (widest > 1 && blocks % widest) widest--;
    if (epilogue != JL_SWIGLU && rows < 512 && k % 256 == 0 && blocks > 8 && widest < 6 && blocks % 8 != 0) {
        const int head = blocks / 8 * 8, tail = blocks - head;
        bool head_ok = false, tail_ok = false;
        int st = skinny_window(ctx, weights, count, X, X16, C, c_f16, rows, ldo, col_offset, epilogue, planes, plane_bytes,
                               other_us, &head_ok, 0, head * 4, true);
        if (st == JL_OK)
            st = skinny_window(ctx, weights, count, X, X16, C, c_f16, rows, ldo, col_offset, JL_RESIDUAL, planes,
                               plane_bytes, other_us, &tail_ok, head * 4, tail * 4, true);
        if (st != JL_OK) return st;
        if (head_ok && tail_ok) {
            st = skinny_window(ctx, weights, count, X, X16, C, c_f16, rows, ldo, col_offset, epilogue, planes, plane_bytes,
                               other_us, taken, 0, head * 4, false);
            if (st != JL_OK) return st;
            return skinny_window(ctx, weights, count, X, X16, C, c_f16, rows, ldo, col_offset, JL_RESIDUAL, planes,
                                 plane_bytes, other_us, taken, head * 4, tail * 4, false);
        }
    }
    return skinny_window(ctx, weights, count, X, X16, C, c_f16, rows, ldo, col_offset, epilogue, planes, plane_bytes,
                         other_us, taken, 0, 0, false);
}
