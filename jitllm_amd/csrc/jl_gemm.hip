// Batched projections (batched decode and batched prefill): C = X . [W0 | W1 | ...]^T on MFMA.
//
// Replaces the reference's dequantise-then-MMA prefill GEMM (gemmMMAQ8 and dequantize*ToFP16,
// J/backend/tornado/kernels/TransformerBatchPrefillKernels.java:917-1076,2325-2363,2397+;
// TransformerComputeKernelsQ4_0.java:85-101; TransformerComputeKernelsQ4_K.java:114-147) and its
// tiled batched-row kernels (matrixVectorTiledBatchQ4_0 / Q4_K, TransformerComputeKernelsQ4_0.java:
// 1205-1292, TransformerComputeKernelsQ4_K.java:1120-1221) with one CDNA4 kernel family:
//
//   * activations are rounded to fp16 once per call (a power-of-two row scale keeps rows with
//     huge magnitudes inside fp16's range and is undone exactly in the epilogue);
//   * weights stay GGUF blocks in HBM; each workgroup decodes the 64-column slice of its weight
//     rows it is about to use into fp16 in LDS -- the value the host tensor's getFloat returns,
//     rounded once to fp16, which is what the reference's dequantize*ToFP16 kernels store;
//   * the contraction runs on v_mfma_f32_16x16x32_f16 with fp32 accumulators;
//   * epilogues: store, residual add, SwiGLU of a gate/up pair; rows past active_rows untouched.
#include <stdlib.h>

#include "jl_device.h"
#include "jl_internal.h"

namespace {

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef _Float16 half4 __attribute__((ext_vector_type(4)));
typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
typedef float floatx4 __attribute__((ext_vector_type(4)));

constexpr int kMaxWeights = 8;

// ---- activations: fp32 -> fp16 with a power-of-two row scale --------------------------------

// One workgroup per row; see jl_row_to_f16.
__global__ void __launch_bounds__(256)
jl_rows_to_f16(const float *__restrict__ X, _Float16 *__restrict__ A, float *__restrict__ row_scale,
               int rows, int k) {
    jl_row_to_f16(X, A, row_scale, rows, k, blockIdx.x);
}

// Activations that arrive as fp16 but in a buffer the kernels cannot read whole row tiles of: the
// active rows copied as they are, the rows that pad the last tile zero-filled.  A thread moves 16 bytes.
__global__ void __launch_bounds__(256)
jl_rows_copy_f16(const _Float16 *__restrict__ X, _Float16 *__restrict__ A, int rows, int k) {
    const int row = blockIdx.x;
    const uint4 *x = (const uint4 *)(X + (int64_t)row * k);
    uint4 *a = (uint4 *)(A + (int64_t)row * k);
    for (int i = threadIdx.x; i < k / 8; i += 256) a[i] = row < rows ? x[i] : uint4{0u, 0u, 0u, 0u};
}

// ---- LDS access by hand ----------------------------------------------------------------------
// Operand tiles arrive by LDS-DMA (global_load_lds_*).  The compiler answers any LDS access it can
// see after such a load with a full vmcnt(0) wait, which would serialise the operand ring, so every
// LDS access of the kernel is inline assembly with its own lgkmcnt wait, the barrier is the bare
// instruction and the vector-memory waits are placed by hand.

typedef __attribute__((address_space(1))) const void gvoid;
typedef __attribute__((address_space(3))) void lvoid;

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

__device__ __forceinline__ half8 lds_read_h8(uint32_t addr) {
    half8 v;
    asm volatile("ds_read_b128 %0, %1\n\ts_waitcnt lgkmcnt(0)" : "=&v"(v) : "v"(addr) : "memory");
    return v;
}

// N 128-bit fragment reads, issued without waiting: the registers are valid only after
// lds_wait_frags() has been given the same arrays.  Nothing may touch them in between.
template <int N>
__device__ __forceinline__ void lds_issue_h8n(const uint32_t (&addr)[N], half8 (&v)[N]) {
    static_assert(N == 2 || N == 4, "fragment batch");
    if constexpr (N == 4) {
        asm volatile(
            "ds_read_b128 %0, %4\n\tds_read_b128 %1, %5\n\tds_read_b128 %2, %6\n\t"
            "ds_read_b128 %3, %7"
            : "=&v"(v[0]), "=&v"(v[1]), "=&v"(v[2]), "=&v"(v[3])
            : "v"(addr[0]), "v"(addr[1]), "v"(addr[2]), "v"(addr[3]) : "memory");
    } else {
        asm volatile("ds_read_b128 %0, %2\n\tds_read_b128 %1, %3"
                     : "=&v"(v[0]), "=&v"(v[1]) : "v"(addr[0]), "v"(addr[1]) : "memory");
    }
}

// Waits until at most LEFT of the fragment reads issued so far are outstanding (LDS reads return
// in order) and hands the given arrays, whose reads are then complete, back to the compiler.
template <int LEFT, int NA, int NBF>
__device__ __forceinline__ void lds_wait_frags_left(half8 (&a)[NA], half8 (&b)[NBF]) {
    static_assert(LEFT == 4 || LEFT == 6 || LEFT == 8, "outstanding reads");
    if constexpr (NA == 4 && NBF == 4) {
        asm volatile("s_waitcnt lgkmcnt(8)"
                     : "+v"(a[0]), "+v"(a[1]), "+v"(a[2]), "+v"(a[3]), "+v"(b[0]), "+v"(b[1]),
                       "+v"(b[2]), "+v"(b[3]) : : "memory");
    } else if constexpr (NA == 4 && NBF == 2) {
        asm volatile("s_waitcnt lgkmcnt(6)"
                     : "+v"(a[0]), "+v"(a[1]), "+v"(a[2]), "+v"(a[3]), "+v"(b[0]), "+v"(b[1])
                     : : "memory");
    } else {
        asm volatile("s_waitcnt lgkmcnt(4)" : "+v"(a[0]), "+v"(a[1]), "+v"(b[0]), "+v"(b[1]) : : "memory");
    }
}

template <int NA, int NBF>
__device__ __forceinline__ void lds_wait_frags(half8 (&a)[NA], half8 (&b)[NBF]) {
    if constexpr (NA == 4 && NBF == 4) {
        asm volatile("s_waitcnt lgkmcnt(0)"
                     : "+v"(a[0]), "+v"(a[1]), "+v"(a[2]), "+v"(a[3]), "+v"(b[0]), "+v"(b[1]),
                       "+v"(b[2]), "+v"(b[3]) : : "memory");
    } else if constexpr (NA == 4 && NBF == 2) {
        asm volatile("s_waitcnt lgkmcnt(0)"
                     : "+v"(a[0]), "+v"(a[1]), "+v"(a[2]), "+v"(a[3]), "+v"(b[0]), "+v"(b[1])
                     : : "memory");
    } else {
        asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(a[0]), "+v"(a[1]), "+v"(b[0]), "+v"(b[1]) : : "memory");
    }
}

// Four 16-byte chunks of one decoded row: chunk i goes to addr ^ (i << 4), i.e. the four stay inside
// one aligned 64-byte group and are permuted by the row's swizzle key already folded into addr.
__device__ __forceinline__ void lds_write_4xh8(uint32_t addr, const half8 (&v)[4]) {
    const uint32_t a1 = addr ^ 16u, a2 = addr ^ 32u, a3 = addr ^ 48u;
    asm volatile(
        "ds_write_b128 %0, %4\n\tds_write_b128 %1, %5\n\tds_write_b128 %2, %6\n\t"
        "ds_write_b128 %3, %7\n\ts_waitcnt lgkmcnt(0)"
        : : "v"(addr), "v"(a1), "v"(a2), "v"(a3), "v"(v[0]), "v"(v[1]), "v"(v[2]), "v"(v[3]) : "memory");
}

__device__ __forceinline__ void lds_read_9dw(uint32_t addr, uint32_t (&w)[9]) {
    uint2 p0, p1, p2, p3;
    uint32_t last;
    asm volatile(
        "ds_read2_b32 %0, %5 offset0:0 offset1:1\n\tds_read2_b32 %1, %5 offset0:2 offset1:3\n\t"
        "ds_read2_b32 %2, %5 offset0:4 offset1:5\n\tds_read2_b32 %3, %5 offset0:6 offset1:7\n\t"
        "ds_read_b32 %4, %5 offset:32\n\ts_waitcnt lgkmcnt(0)"
        : "=&v"(p0), "=&v"(p1), "=&v"(p2), "=&v"(p3), "=&v"(last) : "v"(addr) : "memory");
    w[0] = p0.x; w[1] = p0.y; w[2] = p1.x; w[3] = p1.y; w[4] = p2.x; w[5] = p2.y; w[6] = p3.x;
    w[7] = p3.y; w[8] = last;
}

__device__ __forceinline__ void lds_read_5dw(uint32_t addr, uint32_t (&w)[5]) {
    uint2 p0, p1;
    uint32_t last;
    asm volatile(
        "ds_read2_b32 %0, %3 offset0:0 offset1:1\n\tds_read2_b32 %1, %3 offset0:2 offset1:3\n\t"
        "ds_read_b32 %2, %3 offset:16\n\ts_waitcnt lgkmcnt(0)"
        : "=&v"(p0), "=&v"(p1), "=&v"(last) : "v"(addr) : "memory");
    w[0] = p0.x; w[1] = p0.y; w[2] = p1.x; w[3] = p1.y; w[4] = last;
}

__device__ __forceinline__ void lds_read_3x4(uint32_t a0, uint32_t a1, uint4 &h, uint4 &q0, uint4 &q1) {
    asm volatile(
        "ds_read_b128 %0, %3\n\tds_read_b128 %1, %4\n\tds_read_b128 %2, %4 offset:16\n\t"
        "s_waitcnt lgkmcnt(0)"
        : "=&v"(h), "=&v"(q0), "=&v"(q1) : "v"(a0), "v"(a1) : "memory");
}

// ---- weight decode: raw block bytes -> fp16, two elements per instruction ----------------------
//
// A byte b in 0..255 placed under the exponent byte 0x64 is the fp16 number 1024 + b, exactly; one
// packed subtract recentres it (1152 = 1024 + 128 for a sign-flipped int8, 1032 = 1024 + 8 for a
// nibble), one packed multiply applies the block scale.  Both products are exact before their one
// rounding, so the result is the host's float decode rounded once to fp16.

typedef _Float16 h2 __attribute__((ext_vector_type(2)));

__device__ __forceinline__ h2 bytes_to_h2(uint32_t v, uint32_t sel) {
    // sel picks two bytes of v (selector values 4..7) and pairs each with 0x64 (selector 0)
    return __builtin_bit_cast(h2, __builtin_amdgcn_perm(v, 0x64646464u, sel));
}

// 4 bytes (already in 0..255 "offset" form) -> 4 fp16 = (byte - bias) * d
__device__ __forceinline__ void dword_to_h4(uint32_t v, h2 bias, h2 d, _Float16 *dst) {
    h2 lo = (bytes_to_h2(v, 0x00050004u) - bias) * d;
    h2 hi = (bytes_to_h2(v, 0x00070006u) - bias) * d;
    dst[0] = lo[0];
    dst[1] = lo[1];
    dst[2] = hi[0];
    dst[3] = hi[1];
}

// One thread decodes the 32 elements (row, half) of a 64-wide slice from the raw stage in LDS.
// raw_row = LDS address of the slice's raw bytes (Q8_0 68 B, Q4_0 36 B; Q4_K: 32 nibble bytes, with
// hdr = LDS address of the super-block's 16-byte header and sub = sub-block index 0..7).
template <int TYPE>
__device__ __forceinline__ void decode_half_slice(uint32_t raw_row, uint32_t hdr, int half, int sub,
                                                  half8 (&out)[4]) {
    _Float16 w[32];
    if constexpr (TYPE == JL_Q8_0) {
        // bytes 0..1 scale A | 2..33 quants A | 34..35 scale B | 36..67 quants B
        uint32_t dw[9];
        lds_read_9dw(raw_row + half * 32, dw);
        uint32_t q[8];
        _Float16 d;
        if (half == 0) {
            d = __builtin_bit_cast(_Float16, (unsigned short)(dw[0] & 0xFFFF));
#pragma unroll
            for (int i = 0; i < 8; i++) q[i] = __builtin_amdgcn_alignbit(dw[i + 1], dw[i], 16);
        } else {
            d = __builtin_bit_cast(_Float16, (unsigned short)(dw[0] >> 16));
#pragma unroll
            for (int i = 0; i < 8; i++) q[i] = dw[i + 1];
        }
        const h2 bias = {(_Float16)1152.f, (_Float16)1152.f};
        const h2 dd = {d, d};
#pragma unroll
        for (int i = 0; i < 8; i++) dword_to_h4(q[i] ^ 0x80808080u, bias, dd, &w[4 * i]);
    } else if constexpr (TYPE == JL_Q4_0) {
        // bytes 0..1 scale A | 2..17 nibbles A | 18..19 scale B | 20..35 nibbles B
        uint32_t dw[5];
        lds_read_5dw(raw_row + half * 16, dw);
        uint32_t nb[4];
        _Float16 d;
        if (half == 0) {
            d = __builtin_bit_cast(_Float16, (unsigned short)(dw[0] & 0xFFFF));
#pragma unroll
            for (int i = 0; i < 4; i++) nb[i] = __builtin_amdgcn_alignbit(dw[i + 1], dw[i], 16);
        } else {
            d = __builtin_bit_cast(_Float16, (unsigned short)(dw[0] >> 16));
#pragma unroll
            for (int i = 0; i < 4; i++) nb[i] = dw[i + 1];
        }
        const h2 bias = {(_Float16)1032.f, (_Float16)1032.f};
        const h2 dd = {d, d};
#pragma unroll
        for (int i = 0; i < 4; i++) {
            dword_to_h4(nb[i] & 0x0F0F0F0Fu, bias, dd, &w[4 * i]);              // elements 4i..4i+3
            dword_to_h4((nb[i] >> 4) & 0x0F0F0F0Fu, bias, dd, &w[16 + 4 * i]);  // elements 16+4i..
        }
    } else {
        uint4 h, q0, q1;
        lds_read_3x4(hdr, raw_row, h, q0, q1);
        float d = jl_half_bits_to_float(h.x);
        float dmin = jl_half_bits_to_float(h.x >> 16);
        int sc, mn;
        jl_q4k_scale_min(h.y, h.z, h.w, sub, sc, mn);
        // (d sc) and (dmin m) rounded to fp16, then q * ds - dm in one fused fp16 operation
        const _Float16 ds = (_Float16)(d * (float)sc);
        const _Float16 dm = (_Float16)(dmin * (float)mn);
        const h2 ds2 = {ds, ds}, dm2 = {dm, dm};
        const h2 bias = {(_Float16)1024.f, (_Float16)1024.f};
        const uint32_t qs[8] = {q0.x, q0.y, q0.z, q0.w, q1.x, q1.y, q1.z, q1.w};
        const int shift = (sub & 1) * 4;
#pragma unroll
        for (int i = 0; i < 8; i++) {
            uint32_t v = (qs[i] >> shift) & 0x0F0F0F0Fu;
            h2 lo = (bytes_to_h2(v, 0x00050004u) - bias) * ds2 - dm2;
            h2 hi = (bytes_to_h2(v, 0x00070006u) - bias) * ds2 - dm2;
            w[4 * i + 0] = lo[0];
            w[4 * i + 1] = lo[1];
            w[4 * i + 2] = hi[0];
            w[4 * i + 3] = hi[1];
        }
    }
#pragma unroll
    for (int i = 0; i < 4; i++)
#pragma unroll
        for (int j = 0; j < 8; j++) out[i][j] = w[8 * i + j];
}

// SiLU(g) * u in single precision: g / (1 + exp(-g)) with expf, a few ulp from the host's double
// form and three orders of magnitude inside the fp16 path's tolerance; the double-precision exp
// costs about 150 instructions per output, which matters at T x hidden outputs per call.
__device__ __forceinline__ float gemm_swiglu(float g, float u) {
    return g / (1.0f + __expf(-g)) * u;
}

struct GemmParams {
    const uint8_t *w[kMaxWeights];
    int w_begin[kMaxWeights + 1];  // first virtual output column of each weight
    int count;
    const _Float16 *A;       // [padded_rows x k] fp16
    const float *row_scale;  // [padded_rows]; null: the activations came as fp16, every scale is 1
    float *C;
    int c_f16;               // SWIGLU only: C holds binary16 values, ldo and col_offset count them
    int rows;                // active rows
    int k;
    int n_total;             // virtual output columns (SWIGLU: rows of one weight)
    int64_t ldo;
    int64_t col_offset;
    int epilogue;
    int row_bytes;
    int ntiles, mtiles;      // tile grid (columns, rows)
    int splits;              // K is cut into `splits` equal runs of steps, one workgroup each
    float *partial;          // splits > 1: [splits][mtiles * BM][ntiles * 128] fp32 partial sums
};

constexpr int BN = 128, BK = 64;
constexpr int SUPER = 4;                       // 64-column steps per raw-weight stage (256 columns)
constexpr int W16_STRIDE = 128;                // bytes per decoded row: 64 halfs, chunks XOR-swizzled like A's
constexpr int W16_BYTES = BN * W16_STRIDE;     // 16384

// Raw weight bytes of one row for 256 columns -- always a whole number of 16-byte chunks, and
// 16-byte aligned in the file layout, which is what lets the stage be fetched with 128-bit loads:
// Q8_0 8 blocks = 272 B, Q4_0 8 blocks = 144 B, Q4_K one super-block = 144 B.
template <int TYPE> struct Raw;
template <> struct Raw<JL_Q8_0> { static constexpr int kRowBytes = 272, kStepBytes = 68; };
template <> struct Raw<JL_Q4_0> { static constexpr int kRowBytes = 144, kStepBytes = 36; };
template <> struct Raw<JL_Q4_K> { static constexpr int kRowBytes = 144; };

// Threads that do nothing but issue the LDS-DMA loads of both operands (two waves).
constexpr int kCopyThreads = 128;

// 128-bit loads per copy thread for one raw stage, and the stage's LDS footprint (every load slot
// has a place of its own, including any past the last row)
template <int TYPE> constexpr int raw_loads() { return (BN * Raw<TYPE>::kRowBytes / 16 + kCopyThreads - 1) / kCopyThreads; }
template <int TYPE> constexpr int raw_stage_bytes() { return raw_loads<TYPE>() * kCopyThreads * 16; }

// Activation stages: as many as the 160 KB of LDS leave room for (the Q8_0 raw stages are larger).
template <int TYPE, int BM> constexpr int a_stages() {
    return BM == 128 && TYPE == JL_Q8_0 ? 3 : 5;
}

// Loads that may still be in flight when step s = 4 u + q is awaited (steady state): everything
// issued after the youngest load the step needs.  The copy waves issue, in iteration i (after its
// barrier), first the next raw stage if i % 4 == 0 (RL loads) and then activation step i + AHEAD
// (NLA loads).  Step s needs activation step s (iteration s - AHEAD) and the raw stage of step s + 1
// (iteration 4 u - 4, or 4 u when q == 3).
constexpr int allowed_in_flight(int q, int AHEAD, int NLA, int RL) {
    if (q == 3 && AHEAD > 3) return NLA + 2 * NLA;  // the raw stage opened at q == 0 is the youngest need
    return (AHEAD - 1) * NLA + ((q >= 1 && q < AHEAD) ? RL : 0);
}

template <int TYPE, int BM>
constexpr int gemm_lds_bytes() {
    return 2 * raw_stage_bytes<TYPE>() + a_stages<TYPE, BM>() * BM * 128 + 2 * W16_BYTES;
}

// Workgroup: 640 threads = 10 waves split by role, so that one role's waits are covered by the
// others' work:
//   waves 0-3  *decoders*: turn the raw weight slice of the next step into fp16 in LDS;
//   waves 4-7  *consumers*: read the MFMA fragments and run the matrix pipe;
//   waves 8-9  *copiers*: issue the LDS-DMA loads of both operands and wait for them.  An LDS-DMA
//              load holds its wave at issue while the memory system is busy; in a wave of their
//              own these stalls cost nobody else anything.
// One barrier per 64-column step hands a landed stage from the copiers to the decoders, a decoded
// slice from the decoders to the consumers, and a finished stage back.  Tile BM x 128 outputs:
//   BM = 128: consumer waves 2 (M) x 2 (N), wave tile 64 x 64
//   BM <= 64: consumer waves 1 x 4, wave tile BM x 32
// For JL_SWIGLU the 128 tile columns are 64 gate rows followed by the 64 up rows of the same 64
// outputs; a wave's column blocks are arranged so that it holds gate and up of the same outputs.
//
// Operand movement.  Raw weights: one stage = 128 rows x 256 columns, fetched with 128-bit LDS-DMA
// loads once per four steps (two stages).  Activations: one stage = BM rows x 64 columns of fp16,
// 16-byte chunks XOR-swizzled by row so that fragment reads are bank-conflict free, fetched every
// step (three or four stages).  Decoded weights: two buffers of 128 x 64 fp16.
template <int TYPE, int BM>
__global__ void __launch_bounds__(640) __attribute__((amdgpu_waves_per_eu(3, 3)))
jl_gemm_f16(GemmParams p) {
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    constexpr int RAWB = raw_stage_bytes<TYPE>();
    constexpr int RB = Raw<TYPE>::kRowBytes;
    constexpr int CPR = RB / 16;            // 16-byte chunks per raw row
    constexpr int RL = raw_loads<TYPE>();   // raw loads per thread and stage
    constexpr int NSA = a_stages<TYPE, BM>();
    constexpr int AHEAD = NSA - 1;          // activation steps in flight ahead of the one in use
    constexpr int NLA = BM * 8 / kCopyThreads;  // activation loads per copy thread and step
    constexpr int ABYTES = BM * 128;
    constexpr int WM = BM == 128 ? 2 : 1;
    constexpr int WN = 4 / WM;
    constexpr int TM = BM / WM;       // wave tile rows
    constexpr int TN = BN / WN;       // wave tile columns
    constexpr int MB = TM / 16;       // 16 x 16 blocks per wave along M
    constexpr int NB = TN / 16;
    static_assert(BM == 32 || BM == 64 || BM == 128, "row tile");

    // the role and the wave index are the same for every lane of a wave: keep them in scalar
    // registers so that the pipeline's bookkeeping (and the waits it selects) stays scalar code
    const int wave8 = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const bool decoder = wave8 < 4;
    const bool copier = wave8 >= 8;
    const int tid = threadIdx.x & 255;  // index inside the role (decoders, consumers)
    const int lane = tid & 63;
    const int wave = wave8 & 3;
    const int wm = wave / WN, wn = wave % WN;
    const bool swiglu = p.epilogue == JL_SWIGLU;
    const int cols_per_tile = swiglu ? BN / 2 : BN;
    const int total_tiles = p.ntiles * p.mtiles;
    const int per_xcd = (total_tiles + 7) / 8;
    const int usteps = p.k / (BK * SUPER) / p.splits;  // raw stages (256 columns) per work item
    const int ksteps = usteps * SUPER;

    const uint32_t lds0 = (uint32_t)(uintptr_t)(lvoid *)lds;
    uint8_t *raw_ring = lds;
    uint8_t *a_ring = lds + 2 * RAWB;
    const uint32_t raw0 = lds0;
    const uint32_t a0 = lds0 + 2 * RAWB;
    const uint32_t w16_0 = a0 + NSA * ABYTES;

    // Persistent workgroups: the launch has one workgroup per compute unit (or fewer) and each walks
    // work items wg, wg + G, ... -- a work item is one (tile, split).  Producers run straight on
    // into the next item's first loads while the consumers are still storing the previous tile, so
    // the load latency at the head of a tile and the stores at its tail overlap.
    // Item order: workgroups go to the 8 XCDs round-robin by launch index and each XCD has an L2 of
    // its own, so XCD x takes the x-th contiguous eighth of the tile list, ordered so that the tiles
    // its workgroups hold at any moment are a 4 (row tiles) x 8 (column tiles) patch.
    const int xcd = blockIdx.x & 7;
    const int slot = blockIdx.x >> 3;
    const int slots = (gridDim.x + 7) >> 3;  // workgroups per XCD
    const int items = per_xcd * p.splits;

    // (tile row, tile column, split) of a work item; false when the item is padding
    auto locate = [&](int item, int &mt, int &nt, int &split) -> bool {
        split = item / per_xcd;
        const int logical = xcd * per_xcd + (item - split * per_xcd);
        if (logical >= total_tiles) return false;
        constexpr int GM = 4;
        const int group = logical / (GM * p.ntiles);
        const int rest = logical - group * (GM * p.ntiles);
        const int rows_in_group = p.mtiles - group * GM < GM ? p.mtiles - group * GM : GM;
        nt = rest / rows_in_group;
        mt = group * GM + rest - nt * rows_in_group;
        return true;
    };

    // The roles are separate loops (with the same barriers in the same order) rather than branches
    // inside one loop: a wave only ever runs one of them, and written this way the register
    // allocator sees that their states are never live together.
    //
    // Local step s = 4 u + q uses raw stage u and activation stage s.  The copiers issue
    //   at the head of an item   raw(0), A(0 .. AHEAD - 1)
    //   iteration s              [raw(u + 1) when q == 0]  A(s + AHEAD)     -- after the barrier of s
    // and before the barrier of s they wait until only allowed_in_flight(q) loads are outstanding.
    // The decoders decode step 0 at the head and step s + 1 in iteration s.  Barriers per item: one
    // after the head loads, one per step, one at the end (every LDS read of the item is done before
    // the next item's loads may land).
    static_assert(AHEAD >= 2 && AHEAD <= 4, "the wait table covers 2..4 steps of look-ahead");
    static_assert(AHEAD * NLA + 2 * RL < 64, "outstanding loads must fit the 6-bit counter");

    if (copier) {
        const int ctid = threadIdx.x - 512;   // 0 .. kCopyThreads - 1
        const int cwave = ctid >> 6;
        for (int item = slot; item < items; item += slots) {
            int mt, nt, split;
            if (!locate(item, mt, nt, split)) continue;
            const int m0 = mt * BM;
            const int n0 = nt * cols_per_tile;
            const int ubase = split * usteps;  // first raw stage of this item

            // source row of tile row r (null past the last output column); the weight table is
            // walked with constant indices so that it stays in scalar registers
            auto row_ptr = [&](int r) -> const uint8_t * {
                if (swiglu) {
                    const int vcol = n0 + (r & 63);
                    const uint8_t *base = r >= 64 ? p.w[1] : p.w[0];
                    return vcol < p.n_total ? base + (int64_t)vcol * p.row_bytes : nullptr;
                }
                const int vcol = n0 + r;
                if (vcol >= p.n_total) return nullptr;
                const uint8_t *base = p.w[0];
                int first = 0;
#pragma unroll
                for (int i = 1; i < kMaxWeights; i++) {
                    if (i < p.count && vcol >= p.w_begin[i]) {
                        base = p.w[i];
                        first = p.w_begin[i];
                    }
                }
                return base + (int64_t)(vcol - first) * p.row_bytes;
            };
            // per-thread DMA sources (a slot with nothing to fetch re-reads its own row 0 chunk)
            const uint8_t *wsrc[RL];
            int wstep[RL];  // bytes a slot's source advances per raw stage: RB, or 0 for a dummy slot
#pragma unroll
            for (int j = 0; j < RL; j++) {
                const int i = j * kCopyThreads + ctid;
                const int r = i / CPR;
                const uint8_t *rp = r < BN ? row_ptr(r) : nullptr;
                wstep[j] = rp ? RB : 0;
                wsrc[j] = rp ? rp + (int64_t)ubase * RB + (i - r * CPR) * 16 : p.w[0] + (i & 63) * 16;
            }
            const uint8_t *asrc[NLA];
#pragma unroll
            for (int j = 0; j < NLA; j++) {
                const int i = j * kCopyThreads + ctid;
                const int r = i >> 3, c = i & 7;
                asrc[j] = (const uint8_t *)(p.A + (int64_t)(m0 + r) * p.k + (int64_t)ubase * (BK * SUPER)) +
                          ((c ^ ((r >> 1) & 7)) << 4);
            }
            auto issue_raw = [&](int u) {  // raw stage u (local index) -> ring slot u & 1
                uint8_t *dst = raw_ring + (u & 1) * RAWB;
#pragma unroll
                for (int j = 0; j < RL; j++)
                    __builtin_amdgcn_global_load_lds((gvoid *)(wsrc[j] + (int64_t)u * wstep[j]),
                                                     (lvoid *)(dst + (j * kCopyThreads + cwave * 64) * 16), 16, 0, 0);
            };
            auto issue_a = [&](int s) {  // activation step s (local index) -> ring slot s % NSA
                uint8_t *dst = a_ring + (s % NSA) * ABYTES;
#pragma unroll
                for (int j = 0; j < NLA; j++)
                    __builtin_amdgcn_global_load_lds((gvoid *)(asrc[j] + (int64_t)s * 128),
                                                     (lvoid *)(dst + (j * kCopyThreads + cwave * 64) * 16), 16, 0, 0);
            };

            issue_raw(0);
#pragma unroll
            for (int a = 0; a < AHEAD; a++)
                if (a < ksteps) issue_a(a);
            JL_WAIT_VM(0);
            __builtin_amdgcn_s_barrier();
            for (int s = 0; s < ksteps; s++) {
                const int u = s / SUPER, q = s % SUPER;
                const bool last = u + 1 == usteps;
                // the wait takes an immediate: one case per position inside the raw stage
                if (last) JL_WAIT_VM(0);
                else if (q == 0) JL_WAIT_VM(allowed_in_flight(0, AHEAD, NLA, RL));
                else if (q == 1) JL_WAIT_VM(allowed_in_flight(1, AHEAD, NLA, RL));
                else if (q == 2) JL_WAIT_VM(allowed_in_flight(2, AHEAD, NLA, RL));
                else JL_WAIT_VM(allowed_in_flight(3, AHEAD, NLA, RL));
                __builtin_amdgcn_s_barrier();
                if (q == 0 && !last) issue_raw(u + 1);
                if (s + AHEAD < ksteps) issue_a(s + AHEAD);
            }
            __builtin_amdgcn_s_barrier();
        }
        return;
    }

    if (decoder) {
        const int drow = tid & 127;  // tile row tid % 128, half tid / 128
        const int dhalf = tid >> 7;
        auto dequant = [&](int s) {
            half8 v[4];
            const int u = s / SUPER, q = s % SUPER;
            const uint32_t row = raw0 + (u & 1) * RAWB + drow * RB;
            if constexpr (TYPE == JL_Q4_K)
                decode_half_slice<TYPE>(row + 16 + q * 32, row, dhalf, q * 2 + dhalf, v);
            else
                decode_half_slice<TYPE>(row + q * Raw<TYPE>::kStepBytes, 0, dhalf, 0, v);
            lds_write_4xh8(w16_0 + (s & 1) * W16_BYTES + drow * W16_STRIDE +
                               (((dhalf * 4) ^ ((drow >> 1) & 7)) << 4), v);
        };
        for (int item = slot; item < items; item += slots) {
            int mt, nt, split;
            if (!locate(item, mt, nt, split)) continue;
            __builtin_amdgcn_s_barrier();
            dequant(0);
            for (int s = 0; s < ksteps; s++) {
                __builtin_amdgcn_s_barrier();
                if (s + 1 < ksteps) dequant(s + 1);
            }
            __builtin_amdgcn_s_barrier();
        }
        return;
    }

    // ---- consumers ----
    // their instructions go first: the matrix pipe is what the other roles exist to feed
    __builtin_amdgcn_s_setprio(2);
    // LDS row of each of the wave's column blocks
    int brow[NB];
#pragma unroll
    for (int j = 0; j < NB; j++) {
        if (swiglu) brow[j] = (j / (NB / 2)) * 64 + wn * (TN / 2) + (j % (NB / 2)) * 16;
        else brow[j] = wn * TN + j * 16;
    }
    for (int item = slot; item < items; item += slots) {
        int mt, nt, split;
        if (!locate(item, mt, nt, split)) continue;
        const int m0 = mt * BM;
        const int n0 = nt * cols_per_tile;

        floatx4 acc[MB][NB];
#pragma unroll
        for (int i = 0; i < MB; i++)
#pragma unroll
            for (int j = 0; j < NB; j++) acc[i][j] = floatx4{0.f, 0.f, 0.f, 0.f};

        // A step is two 32-column halves.  The second half's fragment reads are in flight while
        // the first half's MFMAs run.
        half8 fa[2][MB], fb[2][NB];
        auto issue_frags = [&](int s, int ks) {
            const uint32_t abase = a0 + (s % NSA) * ABYTES;
            const uint32_t wbase = w16_0 + (s & 1) * W16_BYTES;
            const int chunk = ks * 4 + (lane >> 4);
            uint32_t aa[MB], ba[NB];
#pragma unroll
            for (int i = 0; i < MB; i++) {
                const int r = wm * TM + i * 16 + (lane & 15);
                aa[i] = abase + r * 128 + ((chunk ^ ((r >> 1) & 7)) << 4);
            }
#pragma unroll
            for (int j = 0; j < NB; j++) {
                const int r = brow[j] + (lane & 15);
                ba[j] = wbase + r * W16_STRIDE + ((chunk ^ ((r >> 1) & 7)) << 4);
            }
            lds_issue_h8n<MB>(aa, fa[ks]);
            lds_issue_h8n<NB>(ba, fb[ks]);
        };
        auto mfma_half = [&](int ks) {
#pragma unroll
            for (int i = 0; i < MB; i++)
#pragma unroll
                for (int j = 0; j < NB; j++)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(fb[ks][j], fa[ks][i], acc[i][j], 0, 0, 0);
        };

        __builtin_amdgcn_s_barrier();
        for (int s = 0; s < ksteps; s++) {
            __builtin_amdgcn_s_barrier();
            // both halves' reads go out at once; the first half's MFMAs start as soon as its own
            // fragments are back (LDS reads return in order)
            issue_frags(s, 0);
            issue_frags(s, 1);
            lds_wait_frags_left<MB + NB>(fa[0], fb[0]);
            mfma_half(0);
            lds_wait_frags<MB, NB>(fa[1], fb[1]);
            mfma_half(1);
        }
        __builtin_amdgcn_s_barrier();

        // ---- epilogue ----
        // The weight fragment went in as the MFMA's row operand, so a lane holds four consecutive
        // output columns 4 * (lane / 16) .. + 3 of activation row lane % 16 of each block: one
        // 16-byte store per block.
        if (p.splits > 1) {
            // partial sums of this run of K: plain 16-byte stores into the scratch plane of this
            // split; jl_gemm_reduce adds the planes in order and applies the epilogue
            const int64_t plane = (int64_t)p.mtiles * BM * p.ntiles * BN;
            float *pp = p.partial + split * plane;
#pragma unroll
            for (int i = 0; i < MB; i++) {
                const int m = m0 + wm * TM + i * 16 + (lane & 15);
                float *prow = pp + (int64_t)m * (p.ntiles * BN) + nt * BN;
#pragma unroll
                for (int j = 0; j < NB; j++) {
                    const int c = brow[j] + (lane >> 4) * 4;  // column inside the 128-wide tile
                    *(float4 *)(prow + c) = float4{acc[i][j][0], acc[i][j][1], acc[i][j][2], acc[i][j][3]};
                }
            }
            continue;
        }
#pragma unroll
        for (int i = 0; i < MB; i++) {
            const int m = m0 + wm * TM + i * 16 + (lane & 15);
            if (m >= p.rows) continue;
            const float rs = p.row_scale ? p.row_scale[m] : 1.f;
            float *crow = p.C + (int64_t)m * p.ldo + p.col_offset;
            if (swiglu) {
#pragma unroll
                for (int j = 0; j < NB / 2; j++) {
                    const int col = n0 + wn * (TN / 2) + j * 16 + (lane >> 4) * 4;
                    float v[4];
#pragma unroll
                    for (int e = 0; e < 4; e++) v[e] = gemm_swiglu(acc[i][j][e] * rs, acc[i][j + NB / 2][e] * rs);
                    if (p.c_f16) {
                        jl_store4_f16((_Float16 *)p.C + (int64_t)m * p.ldo + p.col_offset + col, v, p.n_total - col);
                        continue;
                    }
                    float *dst = crow + col;
                    if (col + 3 < p.n_total && (((uintptr_t)dst) & 15) == 0) {
                        *(float4 *)dst = float4{v[0], v[1], v[2], v[3]};
                    } else {
#pragma unroll
                        for (int e = 0; e < 4; e++)
                            if (col + e < p.n_total) dst[e] = v[e];
                    }
                }
            } else {
#pragma unroll
                for (int j = 0; j < NB; j++) {
                    const int col = n0 + wn * TN + j * 16 + (lane >> 4) * 4;
                    float4 v = {acc[i][j][0] * rs, acc[i][j][1] * rs, acc[i][j][2] * rs, acc[i][j][3] * rs};
                    float *dst = crow + col;
                    if (col + 3 < p.n_total && (((uintptr_t)dst) & 15) == 0) {
                        if (p.epilogue == JL_RESIDUAL) {
                            float4 o = *(const float4 *)dst;
                            v.x += o.x; v.y += o.y; v.z += o.z; v.w += o.w;
                        }
                        *(float4 *)dst = v;
                    } else {
                        const float ve[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
                        for (int e = 0; e < 4; e++) {
                            if (col + e < p.n_total) {
                                if (p.epilogue == JL_RESIDUAL) dst[e] += ve[e];
                                else dst[e] = ve[e];
                            }
                        }
                    }
                }
            }
        }
    }
}

// Sums the split-K planes in split order (so the result does not depend on scheduling) and
// applies row scale and epilogue.  One thread per four consecutive output columns.
__global__ void __launch_bounds__(256)
jl_gemm_reduce(const float *__restrict__ partial, const float *__restrict__ row_scale,
               float *__restrict__ C, int rows, int n_total, int ntiles, int64_t plane, int splits,
               int64_t ldo, int64_t col_offset, int epilogue, int c_f16) {
    const int col = (blockIdx.x * blockDim.x + threadIdx.x) * 4;
    const int m = blockIdx.y;
    if (col >= n_total || m >= rows) return;
    const int64_t width = (int64_t)ntiles * BN;
    float *out = C + (int64_t)m * ldo + col_offset + col;
    const float rs = row_scale ? row_scale[m] : 1.f;
    float v[4];
    if (epilogue == JL_SWIGLU) {
        // tile t holds gate columns 64 t .. 64 t + 63 in its first half and the up columns after
        const int64_t g = (int64_t)m * width + (col >> 6) * BN + (col & 63);
        float4 sg = {0.f, 0.f, 0.f, 0.f}, su = {0.f, 0.f, 0.f, 0.f};
        for (int z = 0; z < splits; z++) {
            const float4 a = *(const float4 *)(partial + z * plane + g);
            const float4 b = *(const float4 *)(partial + z * plane + g + 64);
            sg.x += a.x; sg.y += a.y; sg.z += a.z; sg.w += a.w;
            su.x += b.x; su.y += b.y; su.z += b.z; su.w += b.w;
        }
        v[0] = gemm_swiglu(sg.x * rs, su.x * rs);
        v[1] = gemm_swiglu(sg.y * rs, su.y * rs);
        v[2] = gemm_swiglu(sg.z * rs, su.z * rs);
        v[3] = gemm_swiglu(sg.w * rs, su.w * rs);
        if (c_f16) {
            jl_store4_f16((_Float16 *)C + (int64_t)m * ldo + col_offset + col, v, n_total - col);
            return;
        }
    } else {
        const int64_t g = (int64_t)m * width + col;
        float4 sum = {0.f, 0.f, 0.f, 0.f};
        for (int z = 0; z < splits; z++) {
            const float4 a = *(const float4 *)(partial + z * plane + g);
            sum.x += a.x; sum.y += a.y; sum.z += a.z; sum.w += a.w;
        }
        v[0] = sum.x * rs; v[1] = sum.y * rs; v[2] = sum.z * rs; v[3] = sum.w * rs;
    }
    const bool add = epilogue == JL_RESIDUAL;
    if (col + 3 < n_total && (((uintptr_t)out) & 15) == 0) {
        float4 o = add ? *(const float4 *)out : float4{0.f, 0.f, 0.f, 0.f};
        *(float4 *)out = float4{o.x + v[0], o.y + v[1], o.z + v[2], o.w + v[3]};
    } else {
        for (int e = 0; e < 4 && col + e < n_total; e++) out[e] = add ? out[e] + v[e] : v[e];
    }
}

size_t round_up(size_t v, size_t a) { return (v + a - 1) / a * a; }

}  // namespace

namespace {

// Split-K factor: calls whose tile grid leaves compute units idle cut K across workgroups -- enough
// work items to cover the chip, at least 2 raw stages (512 columns) per split, and partial-sum
// traffic (written once, read once) bounded by the weight bytes: splits * padded_rows <=
// row_bytes / 2.  A divisor of the stage count.
int choose_splits(int rows, int bm, int k, int tiles, int row_bytes, int compute_units, int *unconstrained = nullptr) {
    const int ksteps = k / (BK * SUPER);  // raw stages of 256 columns
    const int padded = (rows + bm - 1) / bm * bm;
    // (the kernel deals each XCD a contiguous eighth of the tiles, rounded up, times the runs: 84
    // tiles are 11 to an XCD, and three runs of each would be 33 work items for its 32 workgroups --
    // two rounds.  Many rows want one round.)
    int want = rows <= 64 ? (2 * compute_units + tiles - 1) / tiles : (compute_units / 8) / ((tiles + 7) / 8);
    int by_steps = ksteps / 2;
    int by_traffic = row_bytes / (2 * padded);
    int s = want < by_steps ? want : by_steps;
    if (by_traffic < s) s = by_traffic;
    if (s < 1) s = 1;
    if (unconstrained) *unconstrained = s;
    while (ksteps % s) s--;
    return s;
}

size_t a16_bytes(int64_t rows, int64_t cols) { return round_up(round_up((size_t)rows, 256) * (size_t)cols * 2, 256); }
size_t scale_bytes(int64_t rows) { return round_up(round_up((size_t)rows, 256) * 4, 256); }

}  // namespace

// Workspace: fp16 activations | row scales | split-K planes.  The planes are bounded by the
// traffic rule in choose_splits: splits * padded_rows <= row_bytes / 2, so splits * padded_rows *
// columns * 4 <= columns * row_bytes * 2 with row_bytes <= 34 * cols / 32.
size_t jl_gemm_workspace_bytes_impl(int64_t max_rows, int64_t cols, int64_t out_cols, int math) {
    if (math == JL_MATH_INT8) return jl_gemm_i8_workspace_bytes(max_rows, cols);
    // (256: the fp16 copy of a call's weights, which calls of a type without a decode-in-the-loop
    // kernel always make, is padded to whole 256-row column tiles)
    size_t planes = round_up(round_up((size_t)out_cols, 256) * (size_t)cols * 17 / 8 + 128 * 128 * 4, 256);
    // calls of 512 rows or more may decode the weights to fp16 once, into the same region (and,
    // for narrow projections, up to eight planes of partial sums: K is cut for 128 x 128 tiles only
    // and into no more work items than twice 256 compute units, which bounds the planes -- their
    // rows are padded to 256, at most twice the tiles' rows); calls of 128 rows or more over a copy
    // the caller keeps cut K the same way.  A call whose workspace is smaller than this keeps K whole.
    if (max_rows >= 128) {
        size_t two = jl_dense_plane_bytes((int)max_rows, (int)out_cols, 8);
        const size_t cap = 2 * (size_t)2 * 256 * 128 * 128 * sizeof(float);
        if (two > cap) two = cap;
        const size_t need = round_up(jl_dense_copy_bytes((int)cols, (int)out_cols), 256) + two;
        if (need > planes) planes = need;
    }
    return a16_bytes(max_rows, cols) + scale_bytes(max_rows) + planes;
}

namespace {

template <int TYPE, int BM>
int launch_gemm(jl_context *ctx, const GemmParams &p, dim3 grid) {
    auto fn = jl_gemm_f16<TYPE, BM>;
    constexpr int lds = gemm_lds_bytes<TYPE, BM>();
    static_assert(lds <= 160 * 1024, "operand rings exceed the 160 KB of LDS");
    static jl_lds_limit_flags configured;
    {
        const int st = jl_raise_lds_limit(configured, ctx->device, (const void *)fn, lds);
        if (st != JL_OK) return st;
    }
    hipLaunchKernelGGL(fn, grid, dim3(640), lds, ctx->stream, p);
    JL_HIP(hipGetLastError());
    return JL_OK;
}

template <int TYPE>
int launch_gemm_type(jl_context *ctx, GemmParams &p, int rows, float *planes, size_t plane_bytes) {
    const int cols_per_tile = p.epilogue == JL_SWIGLU ? BN / 2 : BN;
    p.ntiles = (p.n_total + cols_per_tile - 1) / cols_per_tile;
    const int bm = rows <= 32 ? 32 : rows <= 64 ? 64 : 128;
    p.mtiles = (rows + bm - 1) / bm;
    p.splits = ctx->split_k ? choose_splits(rows, bm, p.k, p.ntiles * p.mtiles, p.row_bytes, ctx->compute_units) : 1;
    const int64_t plane = (int64_t)p.mtiles * bm * p.ntiles * BN;
    if (p.splits > 1 && (size_t)p.splits * plane * 4 > plane_bytes) p.splits = 1;
    p.partial = planes;
    // persistent workgroups, one per compute unit (fewer when there is less work), a multiple of 8
    // so that every XCD runs the same number of them
    // (an XCD's share is an eighth of the tiles rounded up, times the runs: 84 tiles in two runs are
    // 22 work items to an XCD, and a grid of 168 would give it 21 workgroups)
    const int items = (p.ntiles * p.mtiles + 7) / 8 * 8 * p.splits;
    const int wgs = items < ctx->compute_units ? items : ctx->compute_units / 8 * 8;
    const dim3 grid(wgs);
    int st;
    if (bm == 32) st = launch_gemm<TYPE, 32>(ctx, p, grid);
    else if (bm == 64) st = launch_gemm<TYPE, 64>(ctx, p, grid);
    else st = launch_gemm<TYPE, 128>(ctx, p, grid);
    if (st != JL_OK || p.splits == 1) return st;
    hipLaunchKernelGGL(jl_gemm_reduce, dim3((p.n_total + 1023) / 1024, rows), dim3(256), 0, ctx->stream,
                       planes, p.row_scale, p.C, rows, p.n_total, p.ntiles, plane, p.splits, p.ldo,
                       p.col_offset, p.epilogue, p.c_f16);
    JL_HIP(hipGetLastError());
    return JL_OK;
}

}  // namespace

int jl_launch_gemm_reduce(jl_context *ctx, const float *planes, const float *row_scale, float *C, int rows,
                          int n_total, int ntiles, int64_t plane, int splits, int64_t ldo, int64_t col_offset,
                          int epilogue) {
    hipLaunchKernelGGL(jl_gemm_reduce, dim3((n_total + 1023) / 1024, rows), dim3(256), 0, ctx->stream, planes,
                       row_scale, C, rows, n_total, ntiles, plane, splits, ldo, col_offset, epilogue, 0);
    JL_HIP(hipGetLastError());
    return JL_OK;
}

int jl_launch_gemm(jl_context *ctx, const jl_weight *const *weights, int count, const float *X,
                   float *C, int64_t batch, int64_t active_rows, int64_t ldo, int64_t col_offset,
                   int epilogue, int math, void *workspace, size_t workspace_bytes,
                   const jl_resident *resident, const jl_half_io *half) {
    const int type = weights[0]->type;
    const int k = (int)weights[0]->cols;
    if (math == JL_MATH_INT8) {
        // block-scaled int8 arithmetic (Int8GemmKernels): a path of its own; fp16 operands and a
        // resident fp16 copy have no meaning for it
        if (half && half->x16) return jl_fail(JL_ERR_UNSUPPORTED, "jl_gemm: the int8 path takes fp32 activations");
        return jl_launch_gemm_i8(ctx, weights, count, X, C, batch, (int)active_rows, ldo, col_offset, epilogue,
                                 workspace, workspace_bytes);
    }
    if (k % 64 != 0) {
        return jl_fail(JL_ERR_UNSUPPORTED,
                       "jl_gemm: no batched kernel for a row length of %d (a multiple of 64 is needed)", k);
    }
    const _Float16 *X16 = half ? half->x16 : nullptr;
    const bool c_f16 = half && half->c_f16;
    JL_REQUIRE(((uintptr_t)(X16 ? (const void *)X16 : (const void *)X) & 15) == 0 && ((uintptr_t)workspace & 255) == 0,
               "jl_gemm: X must be 16-byte and the workspace 256-byte aligned");
    for (int i = 0; i < count; i++)
        JL_REQUIRE(((uintptr_t)weights[i]->blocks & 15) == 0, "jl_gemm: weight %d is not 16-byte aligned", i);
    // Weights of different types side by side at fewer than 512 rows -- batched decode or a short
    // prompt over a "Q4_K_M" layer's q | k | v, whose v is Q6_K: decoding all of them to fp16 on every
    // call is what a long prompt amortises and a few rows do not.  Without a kept copy such a call is
    // made one run of equal types at a time, each through the kernels its type has, the runs' outputs
    // side by side as one call would leave them.
    if (count > 1 && epilogue != JL_SWIGLU && active_rows < 512 && k % 256 == 0 && !(resident && resident->copy)) {
        bool differ = false;
        for (int i = 1; i < count; i++) differ = differ || weights[i]->type != type;
        if (differ) {
            int64_t at = col_offset;
            for (int i = 0; i < count;) {
                int j = i;
                int64_t width = 0;
                while (j < count && weights[j]->type == weights[i]->type) width += weights[j++]->rows;
                const int st = jl_launch_gemm(ctx, weights + i, j - i, X, C, batch, active_rows, ldo, at, epilogue, math,
                                              workspace, workspace_bytes, nullptr, half);
                if (st != JL_OK) return st;
                at += width;
                i = j;
            }
            return JL_OK;
        }
    }
    const int rows = (int)active_rows;
    // rows are padded to the row tile the kernel will use, never beyond what the workspace holds
    const int padded = (int)round_up((size_t)rows, rows <= 32 ? 32 : rows <= 64 ? 64 : 128);
    // the workspace was sized for `batch` rows, of which `rows` <= batch are converted
    _Float16 *A = (_Float16 *)workspace;
    float *row_scale = (float *)((uint8_t *)workspace + a16_bytes(batch, k));
    const size_t head = a16_bytes(batch, k) + scale_bytes(batch);
    float *planes = (float *)((uint8_t *)workspace + head);
    const size_t plane_bytes = workspace_bytes > head ? workspace_bytes - head : 0;


    // many rows and enough tiles: weights decoded to fp16 once per call, then the plain fp16 GEMM
    int virt = 0;
    for (int i = 0; i < count; i++) virt += (int)weights[i]->rows;
    // A type without a decode-in-the-loop kernel (Q6_K) takes the decode-once path whatever the
    // shape: correct for any row count, tuned for none but prefill.  So do weights of different
    // types in one call (a "Q4_K_M" file's q | k | v with v in Q6_K): each is decoded by its own
    // type, as the reference's prefill projections do (FP16Projections.java:250-330), and the
    // fp16 GEMM does not know the difference.
    bool mixed = false;
    for (int i = 1; i < count; i++) mixed = mixed || weights[i]->type != type;
    // (and so do rows that are whole 64-column steps but not whole 256-column blocks -- 896 columns,
    // the width of the smallest Qwen2.5 -- which the other two kernels' spans and stages cannot cut)
    const bool dense_only = mixed || !jl_has_fused_kernels(type) || k % 256 != 0;
    const size_t copy_bytes = round_up(jl_dense_copy_bytes(k, virt), 256);
    // the decoded copy goes to the caller's resident buffer when there is one that holds it,
    // otherwise to the head of the workspace's third region
    const bool kept = resident && resident->copy && resident->state && resident->bytes >= copy_bytes &&
                      ((uintptr_t)resident->copy & 255) == 0;

    // Calls of 65 .. 511 rows have up to three ways to go, priced per call in microseconds (fitted to
    // graph replays of the calls of a Llama-3.2-1B layer and of 8B-shaped layers at 65 .. 511 rows):
    //   the weight-streaming kernel    its own estimate, which grows with rows x weights
    //   decode in the loop             22 + (Q8_0: 0.30, 4-bit: 0.37) x 128-row tiles x million weights
    //                                  (its cost moves in steps this does not follow beyond 256 rows;
    //                                  with a kept copy it loses to the next way from 192 rows on,
    //                                  every call measured, and is not considered there)
    //   the plain fp16 GEMM            24 + 0.45 x 256-row tiles x million weights over a copy that is
    //                                  kept across calls (from 128 rows); 30 + 2.8 x million weights
    //                                  when the call has to decode first and has no other kernel
    double millions = 0.0, weight_bytes = 0.0;
    for (int i = 0; i < count; i++) {
        millions += (double)weights[i]->rows * k * 1e-6;
        weight_bytes += (double)weights[i]->bytes;
    }
    // (the kernel that decodes in its loop streams no faster than ~1.9 TB/s: the floor of a call over
    // hundreds of MB of Q8_0 at up to 128 rows, a vocabulary projection -- 147 us for 279 MB)
    double in_loop_us = 22.0 + (type == JL_Q8_0 ? 0.30 : 0.37) * ((rows + 127) / 128) * millions;
    if (in_loop_us < weight_bytes / 1.9e6) in_loop_us = weight_bytes / 1.9e6;
    // (that kernel cuts K into equal runs of whole 256-column stages: a stage count with no divisor
    // near the cut it wants -- 43 stages, 11 008 columns: prime -- leaves it a few dozen work items
    // that each walk most of K, and the call takes as many times longer as the runs are too long:
    // measured 137 us where the fit says 39)
    if (rows > 64 && k % 256 == 0) {
        const int tiles = ((virt + 127) / 128) * (((int)rows + 127) / 128);
        int wanted = 1;
        const int got = ctx->split_k ? choose_splits((int)rows, 128, k, tiles, k / jl_block_elems(type) * jl_block_bytes(type),
                                                     ctx->compute_units, &wanted)
                                     : 1;
        if (ctx->split_k && wanted >= 2 * got) in_loop_us = 22.0 + (in_loop_us - 22.0) * wanted / got;
    }
    if (dense_only || (kept && rows >= 192)) in_loop_us = 1e30;
    const double copy_us = kept && rows >= 128 ? 24.0 + 0.45 * ((rows + 255) / 256) * millions
                           : dense_only       ? 30.0 + 2.8 * millions
                                              : 1e30;
    if (rows < 512) {
        // batched decode of up to 64 rows, and calls of up to 511 where it is the cheapest: the
        // weight-streaming kernel reads X itself, fp32 or fp16
        bool taken = false;
        int st = jl_launch_gemm_skinny(ctx, weights, count, X, X16, C, c_f16, rows, ldo, col_offset, epilogue,
                                       planes, plane_bytes, in_loop_us < copy_us ? in_loop_us : copy_us, &taken);
        if (st != JL_OK || taken) return st;
    }

    const size_t in_workspace = kept ? 0 : copy_bytes;
    // (a call that has no other kernel takes the priced tiling at any row count: a few rows over a
    // narrow weight are a few dozen 128 x 128 tiles, and K cut into runs is what fills the chip)
    const int dense_from = dense_only ? 1 : kept && copy_us < in_loop_us ? 128 : 512;
    int dsplits = 1, bm = 256;
    int bn = jl_dense_column_tile(rows, k, virt, epilogue, ctx->compute_units, &dsplits, &bm, dense_from, ctx->split_k);
    if (bn != 0 && dsplits > 1 && in_workspace + jl_dense_plane_bytes(rows, virt, dsplits) > plane_bytes) {
        // no room for the partial sums of a cut K: the cheapest tiling that keeps K whole
        bn = jl_dense_column_tile(rows, k, virt, epilogue, ctx->compute_units, &dsplits, &bm, dense_from, false);
    }
    if (dense_only && bn == 0) {
        bn = 128;
        bm = 256;
        dsplits = 1;
    }
    const bool dense = bn != 0 && in_workspace + (dsplits > 1 ? jl_dense_plane_bytes(rows, virt, dsplits) : 0) <= plane_bytes;
    const int padded_rows = dense ? (int)round_up((size_t)rows, 256) : padded;

    if (dense_only && !dense) {
        if (mixed) {
            return jl_fail(JL_ERR_WORKSPACE, "jl_gemm: weights of mixed types need room for their fp16 copy (%zu bytes) "
                                             "in the workspace", copy_bytes);
        }
        return jl_fail(JL_ERR_WORKSPACE, "jl_gemm: a %s weight needs room for its fp16 copy (%zu bytes) in the workspace",
                       jl_type_name(type), copy_bytes);
    }
    // what a kept copy looks like: gate / up interleaved by half tiles of this BN, or plain
    const int32_t layout = epilogue == JL_SWIGLU ? bn : 1;
    const bool decode = dense && (!kept || *resident->state != layout);
    // a call that decodes its weights converts its fp32 activations in that same launch
    const bool ride_along = decode && !X16;
    if (!X16) {
        if (!ride_along) {
            hipLaunchKernelGGL(jl_rows_to_f16, dim3(padded_rows), dim3(256), 0, ctx->stream, X, A, row_scale, rows, k);
            JL_HIP(hipGetLastError());
        }
    } else {
        // fp16 activations are multiplied as they are (no row scales).  The kernels bring in whole
        // row tiles: the caller's buffer serves directly when its `batch` rows cover the last
        // tile, else the active rows are copied into the workspace and padded with zeros there.
        row_scale = nullptr;
        if ((int64_t)padded_rows <= batch) {
            A = const_cast<_Float16 *>(X16);
        } else {
            hipLaunchKernelGGL(jl_rows_copy_f16, dim3(padded_rows), dim3(256), 0, ctx->stream, X16, A, rows, k);
            JL_HIP(hipGetLastError());
        }
    }
    if (dense) {
        const int st = jl_launch_gemm_dense(ctx, weights, count, A, row_scale, C, rows, ldo, col_offset, epilogue,
                                            kept ? (_Float16 *)resident->copy : (_Float16 *)planes, decode, bm, bn,
                                            dsplits, (float *)((uint8_t *)planes + in_workspace), c_f16,
                                            ride_along ? X : nullptr, ride_along ? row_scale : nullptr);
        if (st == JL_OK && kept) *resident->state = layout;
        return st;
    }

    GemmParams p{};
    p.count = count;
    int begin = 0;
    for (int i = 0; i < count; i++) {
        p.w[i] = weights[i]->blocks;
        p.w_begin[i] = begin;
        begin += (int)weights[i]->rows;
    }
    p.w_begin[count] = begin;
    p.A = A;
    p.row_scale = row_scale;
    p.C = C;
    p.c_f16 = c_f16 ? 1 : 0;
    p.rows = rows;
    p.k = k;
    p.n_total = epilogue == JL_SWIGLU ? (int)weights[0]->rows : begin;
    p.ldo = ldo;
    p.col_offset = col_offset;
    p.epilogue = epilogue;
    p.row_bytes = k / jl_block_elems(type) * jl_block_bytes(type);

    switch (type) {
        case JL_Q8_0: return launch_gemm_type<JL_Q8_0>(ctx, p, rows, planes, plane_bytes);
        case JL_Q4_0: return launch_gemm_type<JL_Q4_0>(ctx, p, rows, planes, plane_bytes);
        case JL_Q4_K: return launch_gemm_type<JL_Q4_K>(ctx, p, rows, planes, plane_bytes);
        default:
            return jl_fail(JL_ERR_UNSUPPORTED, "jl_gemm: no kernel for a ggml type %d weight", type);
    }
}
