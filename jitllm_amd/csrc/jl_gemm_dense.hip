// Batched prefill over many rows: decode the weights to fp16 once per call, then a plain fp16 GEMM.
//
// This is the reference's own two-step shape (dequantize*ToFP16 followed by gemmMMA,
// J/backend/tornado/kernels/TransformerBatchPrefillKernels.java:917-1076,2325-2363): with a
// few hundred or more activation rows the decode is a small fraction of the call when done once, and
// the matrix loop without it affords 256-row tiles and 128 x 64 wave tiles, which halve the LDS
// traffic per flop of the decode-in-the-loop kernel (jl_gemm.hip).  The decoded copy lives in the
// caller's workspace for the duration of the call; in HBM the weights stay GGUF blocks.
//
//   jl_decode_to_f16   raw blocks -> [virtual rows x K] fp16, the host decode rounded once to fp16
//                      (bit for bit what the fused kernel multiplies with); one launch per call
//   jl_gemm_hh<BM, BN> C = A16 . W16^T on v_mfma_f32_16x16x32_f16, BM x BN tiles (256 x 256, 256 x 192,
//                      256 x 128, 128 x 192, 128 x 128) in steps of 64 columns; eight waves that each bring in their
//                      share of both operands by LDS-DMA, the two waves of a SIMD half a step apart
#include "jl_device.h"
#include "jl_internal.h"

namespace {

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef _Float16 h2 __attribute__((ext_vector_type(2)));
typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(1))) const void gvoid;
typedef __attribute__((address_space(3))) void lvoid;

#define JL_WAIT_VM(N) \
    __builtin_amdgcn_s_waitcnt(((N)&0xF) | (((N) >> 4) << 14) | (0x7 << 4) | (0xF << 8))

// ---- weights -> fp16 ---------------------------------------------------------------------------

__device__ __forceinline__ h2 bytes_to_h2(uint32_t v, uint32_t sel) {
    return __builtin_bit_cast(h2, __builtin_amdgcn_perm(v, 0x64646464u, sel));
}

// four bytes in 0..255 offset form -> (byte - bias) * d, four fp16
__device__ __forceinline__ void dword_scaled(uint32_t v, h2 bias, h2 d, h2 &lo, h2 &hi) {
    lo = (bytes_to_h2(v, 0x00050004u) - bias) * d;
    hi = (bytes_to_h2(v, 0x00070006u) - bias) * d;
}

struct DecodeParams {
    const uint8_t *w[8];   // raw blocks of the call's weights
    int begin[9];          // plain layout: weight i fills virtual rows [begin[i], begin[i + 1])
    int count;
    _Float16 *out;         // [ntiles * BN virtual rows x k]
    int k, row_bytes;
    int n_total;           // SWIGLU: rows of one weight
    int half;              // SWIGLU: BN / 2 of the GEMM that will read the copy, else 0; virtual row
                           // t * BN + sel * half + i is row t * half + i of weight sel (0 gate, 1 up)
    int only_own;          // a later pass over weights of mixed types: rows of a weight whose
                           // pointer is null here (another type's, or padding) are left as they are
    // the call's activations, when they ride along (else virtual_rows = the grid's width):
    // workgroups blockIdx.x >= virtual_rows convert activation row blockIdx.x - virtual_rows
    int virtual_rows;
    const float *X;        // [rows x k] fp32
    _Float16 *A;           // [padded rows x k]
    float *row_scale;
    int rows;
};

// eight bytes (two dwords in 0..255 offset form) -> (byte - bias) * d, eight fp16 as one 16-byte store
__device__ __forceinline__ uint4 pack8_scaled(uint32_t q0, uint32_t q1, h2 bias, h2 d) {
    h2 a, b, c, e;
    dword_scaled(q0, bias, d, a, b);
    dword_scaled(q1, bias, d, c, e);
    return uint4{__builtin_bit_cast(uint32_t, a), __builtin_bit_cast(uint32_t, b),
                 __builtin_bit_cast(uint32_t, c), __builtin_bit_cast(uint32_t, e)};
}
__device__ __forceinline__ uint4 pack8_affine(uint32_t q0, uint32_t q1, h2 ds, h2 dm) {
    const h2 bias = {(_Float16)1024.f, (_Float16)1024.f};
    h2 a = (bytes_to_h2(q0, 0x00050004u) - bias) * ds - dm;
    h2 b = (bytes_to_h2(q0, 0x00070006u) - bias) * ds - dm;
    h2 c = (bytes_to_h2(q1, 0x00050004u) - bias) * ds - dm;
    h2 e = (bytes_to_h2(q1, 0x00070006u) - bias) * ds - dm;
    return uint4{__builtin_bit_cast(uint32_t, a), __builtin_bit_cast(uint32_t, b),
                 __builtin_bit_cast(uint32_t, c), __builtin_bit_cast(uint32_t, e)};
}

// One thread decodes 8 consecutive columns of one row into one 16-byte store, so a wave writes
// 1 KB of consecutive fp16 and reads a consecutive run of raw blocks (the 8 quant bytes of a
// Q8_0 / Q4_0 chunk are only 2-byte aligned; the hardware takes unaligned dword loads).
// blockIdx.x is the virtual row -- rows that no weight row fills (the end of the last column tile)
// become zeros -- and blockIdx.y the run of 256 chunks within it.
struct __attribute__((packed, aligned(2))) Quants8 { uint32_t lo, hi; };

template <int TYPE>
__global__ void __launch_bounds__(256) jl_decode_to_f16(DecodeParams p) {
    if ((int)blockIdx.x >= p.virtual_rows) {
        if (blockIdx.y == 0) jl_row_to_f16(p.X, p.A, p.row_scale, p.rows, p.k, blockIdx.x - p.virtual_rows);
        return;
    }
    const int v = blockIdx.x;
    const int c = blockIdx.y * 256 + threadIdx.x;   // chunk of 8 columns
    if (c >= p.k / 8) return;
    uint4 *dst = (uint4 *)(p.out + (int64_t)v * p.k + c * 8);
    // (the table is walked with constant indices so that it stays in scalar registers)
    const uint8_t *w = nullptr;
    int r = 0;
    if (p.half) {
        const int t = v / (2 * p.half), within = v - t * (2 * p.half);
        const int sel = within >= p.half;
        r = t * p.half + within - sel * p.half;
        if (r < p.n_total) w = sel ? p.w[1] : p.w[0];
    } else {
#pragma unroll
        for (int i = 0; i < 8; i++)
            if (i < p.count && v >= p.begin[i] && v < p.begin[i + 1]) {
                w = p.w[i];
                r = v - p.begin[i];
            }
    }
    if (w == nullptr) {
        if (!p.only_own) *dst = uint4{0, 0, 0, 0};
        return;
    }
    const uint8_t *row = w + (int64_t)r * p.row_bytes;
    if constexpr (TYPE == JL_Q8_0) {
        const uint8_t *blk = row + (c >> 2) * 34;
        const _Float16 d = *(const _Float16 *)blk;
        const Quants8 q = *(const Quants8 *)(blk + 2 + (c & 3) * 8);
        const h2 bias = {(_Float16)1152.f, (_Float16)1152.f}, d2 = {d, d};
        *dst = pack8_scaled(q.lo ^ 0x80808080u, q.hi ^ 0x80808080u, bias, d2);
    } else if constexpr (TYPE == JL_Q4_0) {
        // columns 0..15 of a block are the low nibbles of its 16 bytes, 16..31 the high nibbles
        const uint8_t *blk = row + (c >> 2) * 18;
        const _Float16 d = *(const _Float16 *)blk;
        const Quants8 q = *(const Quants8 *)(blk + 2 + (c & 1) * 8);
        const int shift = (c & 2) * 2;
        const h2 bias = {(_Float16)1032.f, (_Float16)1032.f}, d2 = {d, d};
        *dst = pack8_scaled((q.lo >> shift) & 0x0F0F0F0Fu, (q.hi >> shift) & 0x0F0F0F0Fu, bias, d2);
    } else if constexpr (TYPE == JL_Q4_1 || TYPE == JL_Q5_0 || TYPE == JL_IQ4_XS) {
        // chunk c % 4 of the group of 32 c / 4: the low (chunks 0, 1) or high (2, 3) nibbles of
        // eight of the group's sixteen bytes; the value is the host decode in fp32 --
        // (q * d) + m (Q4_1FloatTensor.java:73-94), d * (q - 16) (Q5_0FloatTensor.java:61-85),
        // (d * (ls - 32)) * kvalues[q] (IQ4_XSFloatTensor.java:72-100) -- rounded once to fp16
        const int shift = (c & 2) * 2;
        uint32_t q0, q1;
        float a, b = 0.f;
        if constexpr (TYPE == JL_Q4_1) {
            const uint8_t *blk = row + (c >> 2) * 20;
            const uint32_t dm = *(const uint32_t *)blk;
            q0 = (*(const uint32_t *)(blk + 4 + (c & 1) * 8) >> shift) & 0x0F0F0F0Fu;
            q1 = (*(const uint32_t *)(blk + 8 + (c & 1) * 8) >> shift) & 0x0F0F0F0Fu;
            a = jl_half_bits_to_float(dm);
            b = jl_half_bits_to_float(dm >> 16);
        } else if constexpr (TYPE == JL_Q5_0) {
            const uint8_t *blk = row + (c >> 2) * 22;
            const Quants8 q = *(const Quants8 *)(blk + 6 + (c & 1) * 8);
            const uint32_t qh = (uint32_t)*(const unsigned short *)(blk + 2) |
                                ((uint32_t)*(const unsigned short *)(blk + 4) << 16);
            const uint32_t bits = qh >> (8 * (c & 3));        // the fifth bits of columns 8 (c % 4) ..
            q0 = ((q.lo >> shift) & 0x0F0F0F0Fu) | (jl_spread4(bits) << 4);
            q1 = ((q.hi >> shift) & 0x0F0F0F0Fu) | (jl_spread4(bits >> 4) << 4);
            a = jl_half_bits_to_float(*(const unsigned short *)blk);
        } else {
            const uint8_t *sb = row + (int64_t)(c >> 5) * 136;
            const int g = (c >> 2) & 7;
            const uint2 hdr = *(const uint2 *)sb;
            const uint2 q = *(const uint2 *)(sb + 8 + 16 * g + (c & 1) * 8);
            const int ls = (int)(((hdr.y >> (4 * g)) & 0xFu) | ((((hdr.x >> 16) >> (2 * g)) & 3u) << 4));
            a = jl_mul_rn(jl_half_bits_to_float(hdr.x), (float)(ls - 32));
            q0 = jl_iq4nl_lookup4((q.x >> shift) & 0x0F0F0F0Fu);
            q1 = jl_iq4nl_lookup4((q.y >> shift) & 0x0F0F0F0Fu);
        }
        _Float16 v[8];
#pragma unroll
        for (int e = 0; e < 8; e++) {
            const uint32_t byte = ((e < 4 ? q0 : q1) >> (8 * (e & 3))) & 0xFF;
            float f;
            if constexpr (TYPE == JL_Q4_1) f = __fadd_rn(jl_mul_rn((float)byte, a), b);
            else if constexpr (TYPE == JL_Q5_0) f = jl_mul_rn(a, (float)((int)byte - 16));
            else f = jl_mul_rn(a, (float)(int)(int8_t)byte);
            v[e] = (_Float16)f;
        }
        *dst = *(const uint4 *)v;
    } else if constexpr (TYPE == JL_Q5_K) {
        // chunk c % 32 of super-block c / 32 (d, dmin | 12 scale bytes | qh[32] | qs[128]): sub-block
        // sub, positions pos .. pos + 7; the value is the host decode ((d * sc) * q) - (dmin * m) in
        // fp32 (Q5_KFloatTensor.java:78-122), rounded once to fp16
        const uint8_t *sb = row + (int64_t)(c >> 5) * 176;
        const int sub = (c >> 2) & 7, pos = (c & 3) * 8;
        const uint4 h = *(const uint4 *)sb;
        const uint2 qs = *(const uint2 *)(sb + 48 + (sub >> 1) * 32 + pos);
        const uint2 qh = *(const uint2 *)(sb + 16 + pos);
        int sc, mn;
        jl_q4k_scale_min(h.y, h.z, h.w, sub, sc, mn);
        const float ds = jl_mul_rn(jl_half_bits_to_float(h.x), (float)sc);
        const float dm = jl_mul_rn(jl_half_bits_to_float(h.x >> 16), (float)mn);
        const int nib = (sub & 1) * 4;
        const uint32_t q0 = ((qs.x >> nib) & 0x0F0F0F0Fu) | (((qh.x >> sub) & 0x01010101u) << 4);
        const uint32_t q1 = ((qs.y >> nib) & 0x0F0F0F0Fu) | (((qh.y >> sub) & 0x01010101u) << 4);
        _Float16 v[8];
#pragma unroll
        for (int e = 0; e < 4; e++) {
            v[e] = (_Float16)__fsub_rn(jl_mul_rn(ds, (float)((q0 >> (8 * e)) & 0xFF)), dm);
            v[4 + e] = (_Float16)__fsub_rn(jl_mul_rn(ds, (float)((q1 >> (8 * e)) & 0xFF)), dm);
        }
        *dst = *(const uint4 *)v;
    } else if constexpr (TYPE == JL_Q6_K) {
        // chunk c % 32 of super-block c / 32 (ql[128] | qh[64] | 16 signed scales | d): half h,
        // group g, positions pos .. pos + 7 of the group; the value is the host decode
        // (d * scale) * (q - 32) in fp32 (Q6_KFloatTensor.java:66-122), rounded once to fp16
        const uint8_t *sb = row + (int64_t)(c >> 5) * 210;
        const int e0 = (c & 31) * 8, h = e0 >> 7, g = (e0 >> 5) & 3, pos = e0 & 31;
        const Quants8 ql = *(const Quants8 *)(sb + 64 * h + 32 * (g & 1) + pos);
        const Quants8 qh = *(const Quants8 *)(sb + 128 + 32 * h + pos);
        const float ds = jl_mul_rn(jl_half_bits_to_float(*(const unsigned short *)(sb + 208)),
                                   (float)(int)(int8_t)sb[192 + 8 * h + (pos >> 4) + 2 * g]);
        const int nib = (g >> 1) * 4;
        const uint32_t q0 = ((ql.lo >> nib) & 0x0F0F0F0Fu) | (((qh.lo >> (2 * g)) & 0x03030303u) << 4);
        const uint32_t q1 = ((ql.hi >> nib) & 0x0F0F0F0Fu) | (((qh.hi >> (2 * g)) & 0x03030303u) << 4);
        _Float16 v[8];
#pragma unroll
        for (int e = 0; e < 4; e++) {
            v[e] = (_Float16)jl_mul_rn(ds, (float)((int)((q0 >> (8 * e)) & 0xFF) - 32));
            v[4 + e] = (_Float16)jl_mul_rn(ds, (float)((int)((q1 >> (8 * e)) & 0xFF) - 32));
        }
        *dst = *(const uint4 *)v;
    } else {
        // sub-block c / 4 of super-block c / 32: low nibbles are the even sub-block of a pair of
        // 32 bytes, high nibbles the odd one
        const uint8_t *sb = row + (int64_t)(c >> 5) * 144;
        const int sub = (c >> 2) & 7;
        const uint4 h = *(const uint4 *)sb;
        const uint2 q = *(const uint2 *)(sb + 16 + (sub >> 1) * 32 + (c & 3) * 8);
        const float d = jl_half_bits_to_float(h.x);
        const float dmin = jl_half_bits_to_float(h.x >> 16);
        int sc, mn;
        jl_q4k_scale_min(h.y, h.z, h.w, sub, sc, mn);
        const _Float16 ds = (_Float16)(d * (float)sc), dm = (_Float16)(dmin * (float)mn);
        const int shift = (sub & 1) * 4;
        *dst = pack8_affine((q.x >> shift) & 0x0F0F0F0Fu, (q.y >> shift) & 0x0F0F0F0Fu, h2{ds, ds}, h2{dm, dm});
    }
}

// ---- fp16 GEMM ----------------------------------------------------------------------------------

struct DenseParams {
    const _Float16 *A;       // [padded rows x k]
    const _Float16 *W;       // [ntiles * BN x k], virtual row order
    const float *row_scale;  // null: the activations came as fp16, every scale is 1
    float *C;
    int c_f16;               // SWIGLU only: C holds binary16 values, ldo and col_offset count them
    int rows, k, n_total;    // n_total: output columns (SWIGLU: of one weight)
    int64_t ldo, col_offset;
    int epilogue;
    int ntiles, mtiles;
    int splits;              // K is cut into `splits` equal runs of steps, one work item each
    float *partial;          // splits > 1: [splits][mtiles * BM][ntiles * BN] fp32 partial sums
};

__device__ __forceinline__ float dense_swiglu(float g, float u) { return g * __builtin_amdgcn_rcpf(1.0f + __expf(-g)) * u; }

constexpr int DBK = 64;
constexpr int kRowPad = 256;   // activation rows are padded to whole tiles of the largest row tile

// hands fragment registers whose reads are complete back to the compiler
template <int N>
__device__ __forceinline__ void lds_settle(half8 (&f)[N]) {
    if constexpr (N == 8)
        asm volatile("" : "+v"(f[0]), "+v"(f[1]), "+v"(f[2]), "+v"(f[3]), "+v"(f[4]), "+v"(f[5]), "+v"(f[6]), "+v"(f[7]));
    else if constexpr (N == 6)
        asm volatile("" : "+v"(f[0]), "+v"(f[1]), "+v"(f[2]), "+v"(f[3]), "+v"(f[4]), "+v"(f[5]));
    else if constexpr (N == 4)
        asm volatile("" : "+v"(f[0]), "+v"(f[1]), "+v"(f[2]), "+v"(f[3]));
    else
        asm volatile("" : "+v"(f[0]), "+v"(f[1]));
}

// LDS stage: A rows then W rows, 128 bytes (eight 16-byte chunks) per row; chunk c of row r sits
// at position c ^ ((r >> 1) & 7) -- measured, this pairing of rows lets a 128-bit fragment read of
// 16 rows x 4 chunks run at the full 256 bytes per clock.  A step is 64 columns = two MFMA
// k-blocks: the second block's fragments are read while the first block's MFMAs run, one barrier
// per step.  256 x 256: two stages of 64 KB (the next step's loads are issued right after the
// barrier and have the whole step to land); 256 x 128: three stages of 48 KB; 128 x 128: four of
// 32 KB -- the tile of calls too narrow to give every compute unit a larger one, which would
// otherwise have to cut K across workgroups and pay for a fold.
// (192-column tiles, for projections whose width is a multiple of 192 and not of 256 -- a fused
// q|k|v of 3072 or 6144 columns: 256 x 192 in two stages of 56 KB, 128 x 192 in three of 40 KB)
template <int BM, int BN> constexpr int hh_stages() { return BM + BN >= 448 ? 2 : BM + BN >= 320 ? 3 : 4; }

template <int BM, int BN>
__global__ void __launch_bounds__(512) __attribute__((amdgpu_waves_per_eu(2, 2)))
jl_gemm_hh(DenseParams p) {
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    constexpr int DBM = BM;
    constexpr int WM = BN == 256 ? 2 : 4;     // waves along M
    constexpr int WN = 8 / WM;
    constexpr int TM = DBM / WM, TN = BN / WN;   // wave tile: 128 x 64, 64 x 64, 32 x 64; 64 x 96, 32 x 96
    constexpr int MB = TM / 16, NB = TN / 16;
    constexpr int STAGE = (DBM + BN) * 128;
    constexpr int NS = hh_stages<BM, BN>();
    constexpr int AHEAD = NS - 1;
    constexpr int LA = DBM * 8 / 512;          // 16-byte loads per thread and stage, A part
    constexpr int LW = BN * 8 / 512;
    // Cache prefetch of the weight operand, 256 x 256 tiles: their two-stage ring looks ahead by one
    // step, about a microsecond -- enough for operands that come from the caches, just short for
    // weights that come from HBM, as a model's successive layers' do.  Wave 0 therefore touches 64
    // cache lines (a tile row's 128 bytes of a step each, one 4-byte LDS-DMA load into a spare KB
    // behind the ring) of the step PFD steps past every stage it brings in; the workgroups that
    // share a weight tile take a quarter of its rows each.  Measured on weights from HBM: gate/up
    // at 2048 tokens 126 -> 122 us; with the weights in the memory-side cache it costs 1-2 us, and
    // the smaller tiles (deeper rings, shorter steps) lose more than they gain and go without.
    constexpr int PFW = NS == 2 ? 1 : 0;
    constexpr int PFD = 2;
    static_assert(NB == 4 || NB == 6, "four or six column blocks per wave");
    static_assert(BM == 256 || (BM == 128 && BN <= 192), "row tiles: 256, or 128 with 128 or 192 columns");

    const int tid = threadIdx.x;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int lane = tid & 63;
    const int wm = wave / WN, wn = wave % WN;
    const bool swiglu = p.epilogue == JL_SWIGLU;
    const int cols_per_tile = swiglu ? BN / 2 : BN;
    const int ksteps = p.k / DBK / p.splits;   // steps of one work item
    const uint32_t lds0 = (uint32_t)(uintptr_t)(lvoid *)lds;

    // tile order: XCD x (workgroups blockIdx % 8 == x) takes the x-th eighth of the tiles, walked
    // so that what its workgroups hold at any moment is a patch of few row tiles x many column tiles
    const int total = p.ntiles * p.mtiles;
    const int per_xcd = (total + 7) / 8;
    const int xcd = blockIdx.x & 7, slot = blockIdx.x >> 3, slots = (gridDim.x + 7) >> 3;

    // LDS row of each of the wave's column blocks (SWIGLU: first half of a tile gate, second up)
    int brow[NB];
#pragma unroll
    for (int j = 0; j < NB; j++) {
        if (swiglu) brow[j] = (j / (NB / 2)) * (BN / 2) + wn * (TN / 2) + (j % (NB / 2)) * 16;
        else brow[j] = wn * TN + j * 16;
    }
    // fragment read addresses inside a stage, k-block 0; k-block 1 is the same row, chunk + 4
    const int fr = lane & 15, fg = lane >> 4;
    // (row block i of the wave sits 16 rows = 2048 bytes further on with the same swizzle key, so
    // the A fragments need one address register and immediate offsets)
    uint32_t a_off0, w_off[NB];
    {
        const int r = wm * TM + fr;
        a_off0 = r * 128 + ((fg ^ ((r >> 1) & 7)) << 4);
    }
#pragma unroll
    for (int j = 0; j < NB; j++) {
        const int r = brow[j] + fr;
        w_off[j] = DBM * 128 + r * 128 + ((fg ^ ((r >> 1) & 7)) << 4);
    }

    const uint32_t toff = (uint32_t)(tid >> 3) * (uint32_t)(p.k * 2) + (uint32_t)(((tid & 7) ^ ((tid >> 4) & 7)) << 4);

    for (int item = slot; item < per_xcd * p.splits; item += slots) {
        const int split = item / per_xcd;
        const int logical = xcd * per_xcd + (item - split * per_xcd);
        if (logical >= total) continue;
        const int64_t kbytes = (int64_t)split * ksteps * (DBK * 2);   // first column of this run, in bytes
        constexpr int GM = 4;
        const int group = logical / (GM * p.ntiles);
        const int rest = logical - group * (GM * p.ntiles);
        const int rows_in_group = p.mtiles - group * GM < GM ? p.mtiles - group * GM : GM;
        const int nt = rest / rows_in_group;
        const int mt = group * GM + rest - nt * rows_in_group;
        const int m0 = mt * DBM;

        // this thread's load slots: slot i = 512 n + tid is row i / 8, chunk position i % 8 (source
        // chunk swizzled).  64 n rows do not change the swizzle key and A and W rows are equally
        // long, so one 32-bit thread offset serves every slot on top of a uniform address.
        const uint8_t *a_item = (const uint8_t *)(p.A + (int64_t)m0 * p.k) + kbytes;
        const uint8_t *w_item = (const uint8_t *)(p.W + (int64_t)nt * BN * p.k) + kbytes;
        const int64_t slot_stride = (int64_t)64 * p.k * 2;
        // load n (of LA + LW) of this thread for stage s
        auto issue_one = [&](int s, int n) {
            uint8_t *dst = lds + (s % NS) * STAGE;
            if (n < LA)
                __builtin_amdgcn_global_load_lds((gvoid *)(a_item + n * slot_stride + (int64_t)s * 128 + toff),
                                                 (lvoid *)(dst + (n * 512 + wave * 64) * 16), 16, 0, 0);
            else
                __builtin_amdgcn_global_load_lds((gvoid *)(w_item + (n - LA) * slot_stride + (int64_t)s * 128 + toff),
                                                 (lvoid *)(dst + DBM * 128 + ((n - LA) * 512 + wave * 64) * 16), 16, 0, 0);
        };
        // after stage s's last load (past the last step: its own line again, so that the count of
        // loads per stage does not change)
        // (the GM workgroups that share this weight tile touch a GM-th of its rows each)
        const uint32_t pf_off = (uint32_t)((mt - group * GM) * (BN / GM) + lane % (BN / GM)) * (uint32_t)(p.k * 2);
        auto prefetch = [&](int s) {
            if (wave < PFW) {
                const int ps = s + PFD < ksteps ? s + PFD : ksteps - 1;
                __builtin_amdgcn_global_load_lds((gvoid *)(w_item + (int64_t)ps * 128 + pf_off),
                                                 (lvoid *)(lds + NS * STAGE + wave * 256), 4, 0, 0);
            }
        };
        auto issue = [&](int s) {
#pragma unroll
            for (int n = 0; n < LA + LW; n++) issue_one(s, n);
            prefetch(s);
        };

        floatx4 acc[MB][NB];
#pragma unroll
        for (int i = 0; i < MB; i++)
#pragma unroll
            for (int j = 0; j < NB; j++) acc[i][j] = floatx4{0.f, 0.f, 0.f, 0.f};

        __builtin_amdgcn_s_barrier();   // every LDS read of the previous item is done
#pragma unroll
        for (int a = 0; a < AHEAD; a++)
            if (a < ksteps) issue(a);
        // The two waves of a SIMD (w and w + 4) run half a step apart, so that one of them has
        // MFMAs to issue while the other waits for its fragments: after the barrier of step s the
        // early wave reads the fragments of stage s and then multiplies them; the late wave first
        // multiplies the fragments of stage s - 1, which it holds in registers, and then reads
        // those of stage s.  Both have read stage s when they reach the next barrier.
        half8 fa[2][MB], fb[2][NB];
        auto read_frags = [&](uint32_t base) {
#pragma unroll
            for (int h = 0; h < 2; h++) {
                // k-block h: chunk position of chunk (4 h + fg) is the k-block-0 position ^ (4 h)
#pragma unroll
                for (int j = 0; j < NB; j++)
                    asm volatile("ds_read_b128 %0, %1" : "=&v"(fb[h][j]) : "v"((base + w_off[j]) ^ (h << 6)) : "memory");
                const uint32_t aa = (base + a_off0) ^ (h << 6);
#pragma unroll
                for (int i = 0; i < MB; i++)
                    asm volatile("ds_read_b128 %0, %1 offset:%2" : "=&v"(fa[h][i]) : "v"(aa), "n"(i * 2048) : "memory");
            }
        };
        // The MFMAs of k-block h.  With `loads`, stage `next`'s loads go out between the row
        // blocks, a few at a time: every load occupies the address path for its 1 KB (64 bytes per
        // clock per compute unit, i.e. half the step for a whole stage) and holds its wave at
        // issue while that path is busy, which in one burst would leave the matrix pipe idle.
        auto mfma_block = [&](int h, bool loads, int next) {
            constexpr int PER = (LA + LW + MB - 1) / MB;
#pragma unroll
            for (int i = 0; i < MB; i++) {
#pragma unroll
                for (int j = 0; j < NB; j++)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(fb[h][j], fa[h][i], acc[i][j], 0, 0, 0);
                if (loads) {
#pragma unroll
                    for (int n = i * PER; n < (i + 1) * PER && n < LA + LW; n++) issue_one(next, n);
                    if (i == MB - 1) prefetch(next);
                }
            }
        };
        // stage s landed (this thread's part); the AHEAD - 1 younger stages may be in flight, and in
        // a prefetching wave the line touched after each stage, that of stage s included
        auto stage_ready = [&](int s) {
            const int left = ksteps - 1 - s;
            const int younger = left < AHEAD - 1 ? left : AHEAD - 1;
            if (wave < PFW) {
                if (younger >= 2) JL_WAIT_VM(2 * (LA + LW + 1) + 1);
                else if (younger == 1) JL_WAIT_VM(LA + LW + 2);
                else JL_WAIT_VM(1);
            } else {
                if (younger >= 2) JL_WAIT_VM(2 * (LA + LW));
                else if (younger == 1) JL_WAIT_VM(LA + LW);
                else JL_WAIT_VM(0);
            }
            __builtin_amdgcn_s_barrier();
        };
        // (the slot that stage s + AHEAD goes to held stage s - 1, last read before barrier s)
        if (wave < 4) {
            for (int s = 0; s < ksteps; s++) {
                stage_ready(s);
                const bool more = s + AHEAD < ksteps;
                read_frags(lds0 + (s % NS) * STAGE);
                // LDS reads return in order: the first k-block's MB + NB fragments are back when
                // that many of the second's are still outstanding
                if constexpr (MB + NB == 12) asm volatile("s_waitcnt lgkmcnt(12)" ::: "memory");
                else if constexpr (MB + NB == 10) asm volatile("s_waitcnt lgkmcnt(10)" ::: "memory");
                else if constexpr (MB + NB == 8) asm volatile("s_waitcnt lgkmcnt(8)" ::: "memory");
                else asm volatile("s_waitcnt lgkmcnt(6)" ::: "memory");
                static_assert(MB + NB == 12 || MB + NB == 10 || MB + NB == 8 || MB + NB == 6, "fragments per k-block");
                lds_settle(fa[0]);
                lds_settle(fb[0]);
                mfma_block(0, more, s + AHEAD);
                asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
                lds_settle(fa[1]);
                lds_settle(fb[1]);
                mfma_block(1, false, 0);
            }
        } else {
            auto read_all = [&](int s) {
                read_frags(lds0 + (s % NS) * STAGE);
                asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
                lds_settle(fa[0]);
                lds_settle(fb[0]);
                lds_settle(fa[1]);
                lds_settle(fb[1]);
            };
            stage_ready(0);
            if (AHEAD < ksteps) issue(AHEAD);
            read_all(0);
            for (int s = 1; s < ksteps; s++) {
                stage_ready(s);
                __builtin_amdgcn_s_setprio(2);
                mfma_block(0, s + AHEAD < ksteps, s + AHEAD);
                mfma_block(1, false, 0);
                __builtin_amdgcn_s_setprio(0);
                read_all(s);
            }
            mfma_block(0, false, 0);
            mfma_block(1, false, 0);
        }

        // epilogue: a lane holds four consecutive output columns 4 (lane / 16) .. + 3 of activation
        // row lane % 16 of each block
        const int n0 = nt * cols_per_tile;
        if (p.splits > 1) {
            // partial sums of this run of K: plain 16-byte stores into the plane of this split; the
            // planes are added in split order and the epilogue applied by the reduce kernel
            const int64_t width = (int64_t)p.ntiles * BN;
            float *pp = p.partial + (int64_t)split * p.mtiles * DBM * width;
#pragma unroll
            for (int i = 0; i < MB; i++) {
                const int m = m0 + wm * TM + i * 16 + (lane & 15);
                float *prow = pp + (int64_t)m * width + nt * BN;
#pragma unroll
                for (int j = 0; j < NB; j++) {
                    const int c = brow[j] + (lane >> 4) * 4;
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
                    for (int e = 0; e < 4; e++) v[e] = dense_swiglu(acc[i][j][e] * rs, acc[i][j + NB / 2][e] * rs);
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

template <int BM, int BN>
int launch_dense(jl_context *ctx, const DenseParams &p) {
    auto fn = jl_gemm_hh<BM, BN>;
    constexpr int lds = hh_stages<BM, BN>() * (BM + BN) * 128 + 1024;   // the ring and the prefetch's landing KB
    static jl_lds_limit_flags configured;
    {
        const int st = jl_raise_lds_limit(configured, ctx->device, (const void *)fn, lds);
        if (st != JL_OK) return st;
    }
    // (an XCD's share is an eighth of the tiles rounded up, times the runs of K)
    const int items = (p.ntiles * p.mtiles + 7) / 8 * 8 * p.splits;
    const int wgs = items < ctx->compute_units ? items : ctx->compute_units / 8 * 8;
    hipLaunchKernelGGL(fn, dim3(wgs), dim3(512), lds, ctx->stream, p);
    JL_HIP(hipGetLastError());
    return JL_OK;
}

template <int TYPE>
int launch_decode(jl_context *ctx, const DecodeParams &d, int activation_rows) {
    hipLaunchKernelGGL(jl_decode_to_f16<TYPE>,
                       dim3((unsigned)(d.virtual_rows + activation_rows), (unsigned)((d.k / 8 + 255) / 256)),
                       dim3(256), 0, ctx->stream, d);
    JL_HIP(hipGetLastError());
    return JL_OK;
}

}  // namespace

// Column tile the dense path would use for a call (and in *row_tile the row tile, in *splits the
// runs K is cut into), 0 when the call is not one for it: it takes `min_rows` rows or more (512
// where the call has to decode its weights first) and enough
// work to give most compute units a 128 x 128 tile of an eighth of K.  Every tiling the kernel has
// is priced -- rounds of work items over the compute units x outputs per item x what an output costs
// in that tile, measured with every compute unit busy at K = 2048: 256 x 256 runs at ~1180 TFLOP/s,
// 256 x 192 at ~980, 256 x 128 at ~960, 128 x 192 at ~790, 128 x 128 at ~650 -- and the cheapest
// wins, larger tiles and fewer runs first among equals.  192-column tiles are for widths that are
// whole multiples of them (a fused q|k|v of 3072 or 6144 columns; plain store / residual only).
// 128 x 128 tiles may also cut K into 2, 4 or 8 runs of at least four steps (plain store / residual
// only; not with `may_cut_k` false), which costs the fold's launch and the partial sums' trip
// through memory.
int jl_dense_column_tile(int rows, int k, int out_cols_virtual, int epilogue, int compute_units, int *splits,
                         int *row_tile, int min_rows, bool may_cut_k) {
    *splits = 1;
    *row_tile = 256;
    if (rows < min_rows || k % 64 != 0) return 0;
    const bool swiglu = epilogue == JL_SWIGLU;
    const int64_t small = (int64_t)((rows + 127) / 128) * ((out_cols_virtual + 127) / 128);
    if (small * 8 * 10 < (int64_t)compute_units * 7) return 0;
    // one microsecond in the units below: a 256 x 256 item of 2048 columns takes ~61 us
    const double per_us = 256.0 * 256.0 * 85.0 / 61.0 * 2048.0 / k;
    static const struct { int bm, bn, per_output; } tilings[] = {
        {256, 256, 85}, {256, 192, 100}, {256, 128, 105}, {128, 192, 125}, {128, 128, 150}};
    double best = 0.0;
    int best_bn = 0;
    for (const auto &t : tilings) {
        if (t.bn == 192 && (swiglu || out_cols_virtual % 192 != 0)) continue;
        const int64_t items = (int64_t)((rows + t.bm - 1) / t.bm) * ((out_cols_virtual + t.bn - 1) / t.bn);
        for (int s = 1; s <= 8; s *= 2) {
            if (s > 1 && (!may_cut_k || swiglu || t.bm != 128 || t.bn != 128)) break;
            if ((k / DBK) % s != 0 || k / s < 4 * DBK) break;
            if (s > 1 && items * s > 2 * (int64_t)compute_units) break;   // (bounds the planes: the workspace counts on it)
            // (per XCD: an eighth of the items rounded up, times the runs, over an eighth of the chip)
            const int64_t rounds = ((items + 7) / 8 * s + compute_units / 8 - 1) / (compute_units / 8);
            double cost = (double)rounds * t.bm * t.bn * t.per_output / s;
            // the fold: a launch, and s planes of partial sums written and read back
            if (s > 1) cost += (2.0 + (double)s * rows * out_cols_virtual * 4.0 / 4e6) * per_us;
            if (best_bn == 0 || cost < best * 0.999) {
                best = cost;
                best_bn = t.bn;
                *row_tile = t.bm;
                *splits = s;
            }
        }
    }
    return best_bn;
}

// Bytes of the partial-sum planes of a call that cuts K into `splits` runs (an upper bound: rows
// padded to the largest row tile).
size_t jl_dense_plane_bytes(int rows, int out_cols_virtual, int splits) {
    return (size_t)splits * (size_t)((rows + kRowPad - 1) / kRowPad * kRowPad) * (size_t)((out_cols_virtual + 127) / 128 * 128) * sizeof(float);
}

// Bytes of the decoded copy for `out_cols_virtual` weight rows of `k` columns.
size_t jl_dense_copy_bytes(int k, int out_cols_virtual) {
    return ((size_t)(out_cols_virtual + 255) / 256 * 256) * (size_t)k * 2;
}

int jl_launch_gemm_dense(jl_context *ctx, const jl_weight *const *weights, int count, const _Float16 *A,
                         const float *row_scale, float *C, int rows, int64_t ldo, int64_t col_offset,
                         int epilogue, _Float16 *copy, bool decode, int bm, int bn, int splits, float *planes,
                         bool c_f16, const float *X32, float *row_scale_out) {
    const int type = weights[0]->type;
    const int k = (int)weights[0]->cols;
    const bool swiglu = epilogue == JL_SWIGLU;
    int n_total = 0;
    for (int i = 0; i < (swiglu ? 1 : count); i++) n_total += (int)weights[i]->rows;
    const int cols_per_tile = swiglu ? bn / 2 : bn;
    const int ntiles = (n_total + cols_per_tile - 1) / cols_per_tile;

    if (count > 8) return jl_fail(JL_ERR_UNSUPPORTED, "jl_gemm: more than 8 weights in one call");
    DecodeParams d{};
    for (int i = 0; i < count; i++) {
        d.w[i] = weights[i]->blocks;
        d.begin[i + 1] = d.begin[i] + (int)weights[i]->rows;
    }
    d.count = count;
    d.out = copy;
    d.k = k;
    d.row_bytes = k / jl_block_elems(type) * jl_block_bytes(type);
    d.n_total = n_total;
    d.half = swiglu ? bn / 2 : 0;
    // plain layout: always whole 256-row tiles, so the copy does not depend on the column tile
    // (a copy that is kept across calls stays valid when the row count, hence BN, changes)
    d.virtual_rows = swiglu ? ntiles * bn : (n_total + 255) / 256 * 256;
    // fp32 activations of a call that decodes are converted by the same launch (X32 is null when
    // the caller has converted them, or they came as fp16)
    int xr = 0;
    if (X32) {
        if (!decode) return jl_fail(JL_ERR_INVALID, "jl_gemm: activations handed to a decode that is not due");
        d.X = X32;
        d.A = const_cast<_Float16 *>(A);
        d.row_scale = row_scale_out;
        d.rows = rows;
        xr = (rows + kRowPad - 1) / kRowPad * kRowPad;
    }
    // Each weight is decoded by its own type, as the reference's prefill projections decode theirs
    // (FP16Projections.project, J/backend/tornado/layers/FP16Projections.java:250-330: one decode
    // task per weight, chosen by its dataType()): one pass per type that occurs.  The first pass
    // sees the other types' weights as absent and fills their rows, like the padding, with zeros;
    // the later ones write their own weights' rows only.  The activations ride along once.
    bool first_pass = true;
    for (int i0 = 0; decode && i0 < count; i0++) {
        const int pass_type = weights[i0]->type;
        bool earlier = false;   // decoded by the pass that began at the type's first weight
        for (int j = 0; j < i0; j++) earlier = earlier || weights[j]->type == pass_type;
        if (earlier) continue;
        DecodeParams pass = d;
        for (int j = 0; j < count; j++)
            if (weights[j]->type != pass_type) pass.w[j] = nullptr;
        pass.row_bytes = k / jl_block_elems(pass_type) * jl_block_bytes(pass_type);
        pass.only_own = first_pass ? 0 : 1;
        const int ride = first_pass ? xr : 0;
        first_pass = false;
        int dst;
        switch (pass_type) {
            case JL_Q8_0: dst = launch_decode<JL_Q8_0>(ctx, pass, ride); break;
            case JL_Q4_0: dst = launch_decode<JL_Q4_0>(ctx, pass, ride); break;
            case JL_Q4_K: dst = launch_decode<JL_Q4_K>(ctx, pass, ride); break;
            case JL_Q5_K: dst = launch_decode<JL_Q5_K>(ctx, pass, ride); break;
            case JL_Q6_K: dst = launch_decode<JL_Q6_K>(ctx, pass, ride); break;
            case JL_Q4_1: dst = launch_decode<JL_Q4_1>(ctx, pass, ride); break;
            case JL_Q5_0: dst = launch_decode<JL_Q5_0>(ctx, pass, ride); break;
            case JL_IQ4_XS: dst = launch_decode<JL_IQ4_XS>(ctx, pass, ride); break;
            default: return jl_fail(JL_ERR_UNSUPPORTED, "jl_gemm: no kernel for a ggml type %d weight", pass_type);
        }
        if (dst != JL_OK) return dst;
    }

    DenseParams p{};
    p.A = A;
    p.W = copy;
    p.row_scale = row_scale;
    p.C = C;
    p.c_f16 = c_f16 ? 1 : 0;
    p.rows = rows;
    p.k = k;
    p.n_total = n_total;
    p.ldo = ldo;
    p.col_offset = col_offset;
    p.epilogue = epilogue;
    p.ntiles = ntiles;
    p.mtiles = (rows + bm - 1) / bm;
    p.splits = splits;
    p.partial = planes;
    if (!(bm == 256 || (bm == 128 && bn != 256)) || (bn != 128 && bn != 192 && bn != 256) ||
        (bn == 192 && (swiglu || splits != 1 || n_total % 192 != 0)))
        return jl_fail(JL_ERR_INVALID, "jl_gemm: no %d x %d tile", bm, bn);
    const int st = bn == 256   ? launch_dense<256, 256>(ctx, p)
                   : bn == 192 ? (bm == 256 ? launch_dense<256, 192>(ctx, p) : launch_dense<128, 192>(ctx, p))
                   : bm == 256 ? launch_dense<256, 128>(ctx, p)
                               : launch_dense<128, 128>(ctx, p);
    if (st != JL_OK || splits == 1) return st;
    return jl_launch_gemm_reduce(ctx, planes, row_scale, C, rows, n_total, ntiles,
                                 (int64_t)p.mtiles * bm * ntiles * 128, splits, ldo, col_offset, epilogue);
}
