// Batched prefill on the int8 matrix pipe with one fp32 scale product per 32-block: JL_MATH_INT8.
//
// Replaces the reference's int8 prefill GEMMs -- quantizeActivationsQ8Warp, gemmInt8BlockScaled and
// gemmInt8Q8_0 (J/backend/tornado/kernels/Int8GemmKernels.java:96-129, 270-369, 651-676) -- with
// their arithmetic, which is fixed and explicit (:17-23): activations are quantised per 32-block to
// int8 as round-half-away(x * 127 / amax) with dA = amax / 127; weights are the Q8_0 quants, or the
// Q4_0 nibbles recentred to q - 8, with their fp16 block scale dW widened to fp32; a block's dot
// product is exact in int32, and the output accumulates
//     acc = fma((float) dot * dA, dW, acc)
// over the blocks in k order.  Every step of that is reproduced in that order -- K is never cut --
// so a result equals the CPU statement of the same arithmetic bit for bit.
//
//   jl_quantize_rows_i8   X fp32 [rows x k] -> int8 [padded rows x k], dA as [k / 32][padded rows]
//                         (block-major, so that the 32 rows of a matrix tile are consecutive) and,
//                         for Q4_0, -8 * (sum of the block's int8 activations) in the same layout
//   jl_gemm_i8<TYPE,MI,NJ> v_mfma_i32_32x32x32_i8: one instruction is exactly one 32-block of a
//                         32 x 32 output patch.  The weights are read where they lie: a stage is 64
//                         columns = two blocks = 68 (Q8_0) or 36 (Q4_0) consecutive bytes of every
//                         weight row of the tile, copied into LDS by LDS-DMA as four (two) 16-byte
//                         pieces and one dword per row, piece p of all rows side by side.  A lane
//                         of the weight operand is one weight row and half a block; its 16 quant
//                         bytes are one 16-byte LDS read and one dword, shifted by two bytes for
//                         the even block of a pair (whose quants start 2 bytes into the pair).
//                         Q4_0 nibbles go to the matrix pipe as they are (0..15) and the -8 is the
//                         instruction's own addend: C = -8 * sum(a), a per-row constant.
//
// The matrix pipe is not the bound here.  Each int32 result needs a conversion, a multiply and a
// multiply-add on the vector ALU: 3 lane-operations per 32 multiply-accumulates, against 64
// lane-operations per clock and compute unit, is a sixth of what the int8 MFMA could deliver.
#include "jl_device.h"
#include "jl_internal.h"

namespace {

typedef int intx4 __attribute__((ext_vector_type(4)));
typedef int intx16 __attribute__((ext_vector_type(16)));
typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(1))) const void gvoid;
typedef __attribute__((address_space(3))) void lvoid;

#define JL_WAIT_VM(N) \
    __builtin_amdgcn_s_waitcnt(((N)&0xF) | (((N) >> 4) << 14) | (0x7 << 4) | (0xF << 8))

// ---- activations -> int8 -------------------------------------------------------------------------

// One thread quantises 8 consecutive columns, the four threads of a block share its maximum.
// grid (k / 8 / 256 rounded up, padded rows); rows past `rows` become zeros with a zero scale.
template <bool SUMS>
__global__ void __launch_bounds__(256) jl_quantize_rows_i8(const float *__restrict__ X, int rows, int padded, int k,
                                                           int8_t *__restrict__ A8, float *__restrict__ dA,
                                                           int32_t *__restrict__ sS) {
    const int row = blockIdx.y;
    const int c = blockIdx.x * 256 + threadIdx.x;   // chunk of 8 columns; k / 8 is a multiple of 8
    if (c >= k / 8) return;
    float x[8];
    if (row < rows) {
        const float4 *src = (const float4 *)(X + (int64_t)row * k + c * 8);
        const float4 a = src[0], b = src[1];
        x[0] = a.x; x[1] = a.y; x[2] = a.z; x[3] = a.w; x[4] = b.x; x[5] = b.y; x[6] = b.z; x[7] = b.w;
    } else {
#pragma unroll
        for (int e = 0; e < 8; e++) x[e] = 0.f;
    }
    float amax = 0.f;
#pragma unroll
    for (int e = 0; e < 8; e++) amax = fmaxf(amax, fabsf(x[e]));
    amax = fmaxf(amax, __shfl_xor(amax, 1, 64));
    amax = fmaxf(amax, __shfl_xor(amax, 2, 64));
    const float d = amax / 127.0f;
    const float inv = 127.0f / amax;
    const bool fast = amax >= 4.0e-37f;   // RECIPROCAL_FINITE_AMAX
    uint32_t packed[2] = {0u, 0u};
    int sum = 0;
#pragma unroll
    for (int e = 0; e < 8; e++) {
        int qv = 0;
        if (d > 0.0f) {
            const float v = fast ? jl_mul_rn(x[e], inv) : jl_mul_rn(x[e] / amax, 127.0f);
            qv = (int)floorf(fabsf(v) + 0.5f);
            qv = qv > 127 ? 127 : qv;
            qv = v < 0.0f ? -qv : qv;
        }
        sum += qv;
        packed[e >> 2] |= ((uint32_t)qv & 0xFFu) << (8 * (e & 3));
    }
    *(uint2 *)(A8 + (int64_t)row * k + c * 8) = uint2{packed[0], packed[1]};
    if constexpr (SUMS) {
        sum += __shfl_xor(sum, 1, 64);
        sum += __shfl_xor(sum, 2, 64);
    }
    if ((c & 3) == 0) {
        const int64_t at = (int64_t)(c >> 2) * padded + row;
        dA[at] = d;
        if constexpr (SUMS) sS[at] = -8 * sum;
    }
}

// ---- the GEMM --------------------------------------------------------------------------------------

constexpr int kMaxSeg = 8;

struct I8Params {
    const int8_t *A8;       // [padded rows x k]
    const float *dA;        // [k / 32][padded rows]
    const int32_t *sS;      // Q4_0: [k / 32][padded rows], -8 * sum of the block's activations
    const uint8_t *w[kMaxSeg];
    int seg_rows[kMaxSeg];
    int seg_tile_begin[kMaxSeg + 1];   // first column tile of each weight; [nseg] = all tiles
    int seg_col_begin[kMaxSeg];        // first output column of each weight
    int nseg;
    const uint8_t *w_up;    // JL_SWIGLU: the up weight
    float *C;
    int rows, padded, k;
    int64_t ldo, col_offset;
    int epilogue;
    int row_bytes;
    int ntiles, mtiles;
};

template <int TYPE> struct Raw {
    static constexpr int kPair = TYPE == JL_Q8_0 ? 68 : 36;   // bytes of two blocks
    static constexpr int kPlanes = TYPE == JL_Q8_0 ? 4 : 2;   // 16-byte pieces of a pair; one dword follows
};

__device__ __forceinline__ float i8_swiglu(float g, float u) { return (g / (1.0f + __expf(-g))) * u; }

// Workgroup = 2 x 2 waves, each a patch of MI x NJ MFMA tiles of 32 x 32: a tile of BM = 64 MI
// activation rows x BN = 64 NJ weight rows (128 x 128 or 64 x 64).  JL_SWIGLU: the weight rows of a
// tile are 32-row runs of gate rows and of the up rows of the same outputs in turn -- a wave with
// two column patches holds both halves of an output in one lane, waves with one exchange them
// through LDS at the end.
template <int TYPE, int MI, int NJ>
__global__ void __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2, MI == 2 ? 2 : 4)))
jl_gemm_i8(I8Params p) {
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    constexpr int WM = 2, WN = 2, NW = 4;
    constexpr int BM = 32 * MI * WM, BN = 32 * NJ * WN;
    constexpr int PAIR = Raw<TYPE>::kPair, NP = Raw<TYPE>::kPlanes;
    constexpr bool Q4 = TYPE == JL_Q4_0;
    // stage layout
    constexpr int A_OFF = 0;
    constexpr int W_OFF = BM * 64;
    constexpr int WD_OFF = W_OFF + NP * BN * 16;
    constexpr int SA_OFF = WD_OFF + BN * 4;
    constexpr int S_REGION = 8 * BM < 1024 ? 1024 : 8 * BM;   // a wave-wide 16-byte load fills 1 KB
    constexpr int SS_OFF = SA_OFF + S_REGION;
    constexpr int STAGE = SS_OFF + (Q4 ? S_REGION : 0);
    constexpr int NS = 3, AHEAD = NS - 1;
    // loads of one wave and stage
    constexpr int LA = MI;                       // 16-byte loads of the activation tile
    constexpr int LW = (NP * NJ + NW - 1) / NW;  // 16-byte loads of the weight pieces (waves repeat
                                                 // one another's when there are fewer than four)
    constexpr int NL = LA + LW + 1 + 1 + (Q4 ? 1 : 0);

    const int tid = threadIdx.x;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int lane = tid & 63;
    const int wm = wave / WN, wn = wave % WN;
    const int l = lane & 31, h = lane >> 5;
    const bool swiglu = p.epilogue == JL_SWIGLU;
    const uint32_t lds0 = (uint32_t)(uintptr_t)(lvoid *)lds;

    // tile of this workgroup: XCD x (workgroups with blockIdx % 8 == x) takes the x-th eighth of the
    // tiles, row tiles fastest, so that the workgroups resident on an XCD share few column tiles
    const int total = p.ntiles * p.mtiles;
    const int per_xcd = (total + 7) / 8;
    const int logical = (blockIdx.x & 7) * per_xcd + (blockIdx.x >> 3);
    if ((int)(blockIdx.x >> 3) >= per_xcd || logical >= total) return;
    const int nt = logical / p.mtiles, mt = logical - nt * p.mtiles;
    const int m0 = mt * BM;
    const int ksteps = p.k / 64;

    // the weight of this column tile (constant indices keep the table in scalar registers)
    const uint8_t *seg_w = p.w[0];
    int seg_rows = p.seg_rows[0], seg_tile0 = 0, seg_col0 = 0;
#pragma unroll
    for (int i = 1; i < kMaxSeg; i++) {
        if (i < p.nseg && nt >= p.seg_tile_begin[i]) {
            seg_w = p.w[i];
            seg_rows = p.seg_rows[i];
            seg_tile0 = p.seg_tile_begin[i];
            seg_col0 = p.seg_col_begin[i];
        }
    }
    // first byte of the weight row behind row r of the tile's weight operand; rows past the
    // weight's last re-read its last row (their results are never stored)
    auto weight_row = [&](int r) -> const uint8_t * {
        const uint8_t *w = seg_w;
        int row;
        if (swiglu) {
            w = ((r >> 5) & 1) ? p.w_up : seg_w;           // (JL_SWIGLU runs with NJ == 2)
            row = nt * (BN / 2) + 32 * (r >> 6) + (r & 31);
        } else {
            row = (nt - seg_tile0) * BN + r;
        }
        row = row < seg_rows ? row : seg_rows - 1;
        return w + (int64_t)row * p.row_bytes;
    };

    // ---- this wave's loads: a global address per lane and a uniform LDS offset each; a stage
    // advances every address by a constant
    const uint8_t *src[NL];
    int step[NL];
    uint32_t dst[NL];
    {
        int n = 0;
#pragma unroll
        for (int j = 0; j < LA; j++, n++) {
            const int s = (wave * LA + j) * 64 + lane;        // slot: row s / 4, position s % 4
            const int row = s >> 2, pos = s & 3;
            const int chunk = pos ^ ((row >> 2) & 3);
            src[n] = (const uint8_t *)p.A8 + (int64_t)(m0 + row) * p.k + chunk * 16;
            step[n] = 64;
            dst[n] = A_OFF + (wave * LA + j) * 1024;
        }
#pragma unroll
        for (int j = 0; j < LW; j++, n++) {
            const int q = (wave * LW + j) % (NP * NJ);         // piece q / NJ, rows 64 (q % NJ) ..
            const int piece = q / NJ, r0 = 64 * (q % NJ);
            src[n] = weight_row(r0 + lane) + piece * 16;
            step[n] = PAIR;
            dst[n] = W_OFF + piece * BN * 16 + r0 * 16;
        }
        {
            const int r0 = 64 * (wave % NJ);                   // the dword behind the pieces
            src[n] = weight_row(r0 + lane) + NP * 16;
            step[n] = PAIR;
            dst[n] = WD_OFF + r0 * 4;
            n++;
        }
        {
            // the stage's two blocks of BM scales: slot s = block s / (BM / 4), rows 4 (s % (BM / 4)) ..;
            // lanes past the last slot repeat an earlier one into the padding behind the scales
            const int s = lane % (BM / 2);
            const int b = s / (BM / 4), r4 = s % (BM / 4);
            const int64_t at = ((int64_t)b * p.padded + m0 + 4 * r4) * 4;
            src[n] = (const uint8_t *)p.dA + at;
            step[n] = 2 * p.padded * 4;
            dst[n] = SA_OFF;
            n++;
            if constexpr (Q4) {
                src[n] = (const uint8_t *)p.sS + at;
                step[n] = 2 * p.padded * 4;
                dst[n] = SS_OFF;
                n++;
            }
        }
    }
    auto issue = [&](int s) {
        uint8_t *base = lds + (s % NS) * STAGE;
#pragma unroll
        for (int n = 0; n < NL; n++) {
            const uint8_t *g = src[n] + (int64_t)s * step[n];
            if (n == LA + LW) __builtin_amdgcn_global_load_lds((gvoid *)g, (lvoid *)(base + dst[n]), 4, 0, 0);
            else __builtin_amdgcn_global_load_lds((gvoid *)g, (lvoid *)(base + dst[n]), 16, 0, 0);
        }
    };

    // ---- fragment addresses inside a stage
    // activations: row wm 32 MI + mi 32 + l, 16-byte chunk 2 b + h at position chunk ^ ((row >> 2) & 3)
    uint32_t a_addr[2];
#pragma unroll
    for (int b = 0; b < 2; b++) a_addr[b] = A_OFF + (wm * 32 * MI + l) * 64 + (((2 * b + h) ^ ((l >> 2) & 3)) << 4);
    const uint32_t s_addr = (wm * 32 * MI + 4 * h) * 4;    // + block * BM * 4 + mi * 128 + g * 32
    // weights: row r = wn 32 NJ + nj 32 + l.  Even block: the quants are bytes 2 + 16 h .. of the pair,
    // piece h from byte 2 on and the first two bytes of piece h + 1; odd block: bytes 36 + 16 h ..
    // (Q8_0; 20 .. for Q4_0, both halves), the last three dwords of a piece and the first of the next.
    const int wr = wn * 32 * NJ + l;
    uint32_t w1[2], w2[2], w3[2];
    if constexpr (!Q4) {
        w1[0] = W_OFF + h * BN * 16 + wr * 16;
        w2[0] = W_OFF + (h + 1) * BN * 16 + wr * 16;
        w3[0] = W_OFF + wr * 16;                        // scale: low half of the pair's first dword
        w1[1] = W_OFF + (2 + h) * BN * 16 + wr * 16;
        w2[1] = h ? WD_OFF + wr * 4 : W_OFF + 3 * BN * 16 + wr * 16;
        w3[1] = W_OFF + 2 * BN * 16 + wr * 16;          // scale: high half of byte 32..35
    } else {
        w1[0] = W_OFF + wr * 16;
        w2[0] = W_OFF + BN * 16 + wr * 16;
        w3[0] = 0;
        w1[1] = W_OFF + BN * 16 + wr * 16;
        w2[1] = WD_OFF + wr * 4;
        w3[1] = 0;
    }

    floatx4 acc[MI][NJ][4];
#pragma unroll
    for (int mi = 0; mi < MI; mi++)
#pragma unroll
        for (int nj = 0; nj < NJ; nj++)
#pragma unroll
            for (int g = 0; g < 4; g++) acc[mi][nj][g] = floatx4{0.f, 0.f, 0.f, 0.f};

#pragma unroll
    for (int a = 0; a < AHEAD; a++)
        if (a < ksteps) issue(a);

    for (int s = 0; s < ksteps; s++) {
        // stage s has landed (this wave's part); younger stages may stay in flight
        if (s + 1 < ksteps) JL_WAIT_VM(NL * (AHEAD - 1));
        else JL_WAIT_VM(0);
        __builtin_amdgcn_s_barrier();
        // the slot stage s + AHEAD goes to held stage s - 1, which every wave has finished reading
        if (s + AHEAD < ksteps) issue(s + AHEAD);
        const uint32_t base = lds0 + (s % NS) * STAGE;
#pragma unroll
        for (int b = 0; b < 2; b++) {
            intx4 fa[MI], fb[NJ];
            floatx4 da[MI][4];
            intx4 ss[MI][4];
            float dw[NJ];
            // -- reads (by hand: the compiler would wait for the LDS-DMA loads before any LDS
            // access it can see)
#pragma unroll
            for (int mi = 0; mi < MI; mi++) {
                asm volatile("ds_read_b128 %0, %1 offset:%2" : "=&v"(fa[mi]) : "v"(base + a_addr[b]), "n"(mi * 2048) : "memory");
#pragma unroll
                for (int g = 0; g < 4; g++) {
                    asm volatile("ds_read_b128 %0, %1 offset:%2" : "=&v"(da[mi][g])
                                 : "v"(base + SA_OFF + b * BM * 4 + s_addr), "n"(mi * 128 + g * 32) : "memory");
                    if constexpr (Q4)
                        asm volatile("ds_read_b128 %0, %1 offset:%2" : "=&v"(ss[mi][g])
                                     : "v"(base + SS_OFF + b * BM * 4 + s_addr), "n"(mi * 128 + g * 32) : "memory");
                }
            }
            intx4 r1[NJ];
            uint32_t r2[NJ], r3[NJ];
#pragma unroll
            for (int nj = 0; nj < NJ; nj++) {
                asm volatile("ds_read_b128 %0, %1 offset:%2" : "=&v"(r1[nj]) : "v"(base + w1[b]), "n"(nj * 512) : "memory");
                // (the dword plane has 4-byte rows: 32 rows on are 128 bytes, not 512)
                if (b == 1) {
                    uint32_t a2 = base + w2[1] + nj * ((Q4 || h) ? 128 : 512);
                    asm volatile("ds_read_b32 %0, %1" : "=&v"(r2[nj]) : "v"(a2) : "memory");
                } else {
                    asm volatile("ds_read_b32 %0, %1 offset:%2" : "=&v"(r2[nj]) : "v"(base + w2[0]), "n"(nj * 512) : "memory");
                }
                if constexpr (!Q4)
                    asm volatile("ds_read_b32 %0, %1 offset:%2" : "=&v"(r3[nj]) : "v"(base + w3[b]), "n"(nj * 512) : "memory");
            }
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
#pragma unroll
            for (int nj = 0; nj < NJ; nj++) {
                asm volatile("" : "+v"(r1[nj]), "+v"(r2[nj]));
                if constexpr (!Q4) asm volatile("" : "+v"(r3[nj]));
            }
#pragma unroll
            for (int mi = 0; mi < MI; mi++) {
                asm volatile("" : "+v"(fa[mi]), "+v"(da[mi][0]), "+v"(da[mi][1]), "+v"(da[mi][2]), "+v"(da[mi][3]));
                if constexpr (Q4) asm volatile("" : "+v"(ss[mi][0]), "+v"(ss[mi][1]), "+v"(ss[mi][2]), "+v"(ss[mi][3]));
            }
            // -- the weight operand and its scale
#pragma unroll
            for (int nj = 0; nj < NJ; nj++) {
                intx4 q;
                if (b == 0) {
                    q[0] = (int)__builtin_amdgcn_alignbit((uint32_t)r1[nj][1], (uint32_t)r1[nj][0], 16);
                    q[1] = (int)__builtin_amdgcn_alignbit((uint32_t)r1[nj][2], (uint32_t)r1[nj][1], 16);
                    q[2] = (int)__builtin_amdgcn_alignbit((uint32_t)r1[nj][3], (uint32_t)r1[nj][2], 16);
                    q[3] = (int)__builtin_amdgcn_alignbit(r2[nj], (uint32_t)r1[nj][3], 16);
                } else {
                    q[0] = r1[nj][1];
                    q[1] = r1[nj][2];
                    q[2] = r1[nj][3];
                    q[3] = (int)r2[nj];
                }
                if constexpr (Q4) {
                    // the block's 16 bytes hold columns 0..15 in their low and 16..31 in their high
                    // nibbles: lane half h takes nibble h of every byte, as the values 0..15
                    const int sh = 4 * h;
#pragma unroll
                    for (int e = 0; e < 4; e++) q[e] = (int)(((uint32_t)q[e] >> sh) & 0x0F0F0F0Fu);
                    dw[nj] = jl_half_bits_to_float(b == 0 ? (uint32_t)r1[nj][0] : (uint32_t)r1[nj][0] >> 16);
                } else {
                    dw[nj] = jl_half_bits_to_float(b == 0 ? r3[nj] : r3[nj] >> 16);
                }
                fb[nj] = q;
            }
            // -- one MFMA per 32 x 32 patch and block, then (float) dot * dA, fused-multiplied by dW
            // into the accumulator: register 4 g + j of a patch is activation row 8 g + 4 h + j
            intx16 dot[MI][NJ];
#pragma unroll
            for (int nj = 0; nj < NJ; nj++)
#pragma unroll
                for (int mi = 0; mi < MI; mi++) {
                    intx16 c;
#pragma unroll
                    for (int i = 0; i < 16; i++) c[i] = Q4 ? ss[mi][i >> 2][i & 3] : 0;
                    dot[mi][nj] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa[mi], fb[nj], c, 0, 0, 0);
                }
#pragma unroll
            for (int nj = 0; nj < NJ; nj++)
#pragma unroll
                for (int mi = 0; mi < MI; mi++)
#pragma unroll
                    for (int i = 0; i < 16; i++) {
                        const float t = (float)dot[mi][nj][i] * da[mi][i >> 2][i & 3];
                        acc[mi][nj][i >> 2][i & 3] = __builtin_fmaf(t, dw[nj], acc[mi][nj][i >> 2][i & 3]);
                    }
        }
    }

    // ---- epilogue: a lane holds one output column and 16 activation rows of each patch
#pragma unroll
    for (int mi = 0; mi < MI; mi++) {
#pragma unroll
        for (int nj = 0; nj < NJ; nj++) {
            if (swiglu && nj == 1) continue;
            int col, limit;
            if (swiglu) {
                col = nt * (BN / 2) + 32 * wn + l;
                limit = seg_rows;
            } else {
                col = (nt - seg_tile0) * BN + wn * 32 * NJ + nj * 32 + l;
                limit = seg_rows;
            }
            if (col >= limit) continue;
            float *cbase = p.C + p.col_offset + seg_col0 + col;
#pragma unroll
            for (int i = 0; i < 16; i++) {
                const int m = m0 + wm * 32 * MI + mi * 32 + 8 * (i >> 2) + 4 * h + (i & 3);
                if (m >= p.rows) continue;
                float *dstp = cbase + (int64_t)m * p.ldo;
                const float v = acc[mi][nj][i >> 2][i & 3];
                if (swiglu) *dstp = i8_swiglu(v, acc[mi][NJ - 1][i >> 2][i & 3]);
                else if (p.epilogue == JL_RESIDUAL) *dstp += v;
                else *dstp = v;
            }
        }
    }
}

template <int TYPE, int MI, int NJ>
int launch_i8(jl_context *ctx, const I8Params &p) {
    auto fn = jl_gemm_i8<TYPE, MI, NJ>;
    constexpr int BM = 64 * MI, BN = 64 * NJ;
    constexpr int region = 8 * BM < 1024 ? 1024 : 8 * BM;
    constexpr int stage = BM * 64 + Raw<TYPE>::kPlanes * BN * 16 + BN * 4 + region * (TYPE == JL_Q4_0 ? 2 : 1);
    constexpr int lds = 3 * stage;
    static jl_lds_limit_flags configured;
    {
        const int st = jl_raise_lds_limit(configured, ctx->device, (const void *)fn, lds);
        if (st != JL_OK) return st;
    }
    const int total = p.ntiles * p.mtiles;
    const int grid = (total + 7) / 8 * 8;
    hipLaunchKernelGGL(fn, dim3(grid), dim3(256), lds, ctx->stream, p);
    JL_HIP(hipGetLastError());
    return JL_OK;
}

template <int TYPE>
int launch_i8_tile(jl_context *ctx, const I8Params &p, int bm, int bn) {
    if (bm == 128) return launch_i8<TYPE, 2, 2>(ctx, p);
    return bn == 128 ? launch_i8<TYPE, 1, 2>(ctx, p) : launch_i8<TYPE, 1, 1>(ctx, p);
}

size_t round_up(size_t v, size_t a) { return (v + a - 1) / a * a; }

}  // namespace

// Workspace of the int8 path: quantised activations | their scales | (Q4_0) their block sums, for
// `max_rows` rows padded to whole 128-row tiles.
size_t jl_gemm_i8_workspace_bytes(int64_t max_rows, int64_t cols) {
    const size_t padded = round_up((size_t)max_rows, 128);
    return round_up(padded * (size_t)cols, 256) + 2 * round_up(padded * (size_t)(cols / 32) * 4, 256);
}

int jl_launch_gemm_i8(jl_context *ctx, const jl_weight *const *weights, int count, const float *X, float *C,
                      int64_t batch, int rows, int64_t ldo, int64_t col_offset, int epilogue, void *workspace,
                      size_t workspace_bytes) {
    const int type = weights[0]->type;
    const int k = (int)weights[0]->cols;
    if (type != JL_Q8_0 && type != JL_Q4_0) {
        return jl_fail(JL_ERR_UNSUPPORTED, "jl_gemm: no int8 kernel for a %s weight (Q8_0 and Q4_0 have one)",
                       jl_type_name(type));
    }
    if (k % 64 != 0) {
        return jl_fail(JL_ERR_UNSUPPORTED, "jl_gemm: the int8 kernel needs a row length that is a multiple of 64, not %d", k);
    }
    if (count > kMaxSeg) return jl_fail(JL_ERR_UNSUPPORTED, "jl_gemm: more than 8 weights in one call");
    JL_REQUIRE(((uintptr_t)X & 15) == 0 && ((uintptr_t)workspace & 255) == 0,
               "jl_gemm: X must be 16-byte and the workspace 256-byte aligned");
    for (int i = 0; i < count; i++)
        JL_REQUIRE(((uintptr_t)weights[i]->blocks & 3) == 0, "jl_gemm: weight %d is not 4-byte aligned", i);
    if (workspace_bytes < jl_gemm_i8_workspace_bytes(batch, k)) {
        return jl_fail(JL_ERR_WORKSPACE, "jl_gemm: the int8 path needs a workspace of %zu bytes, %zu given",
                       jl_gemm_i8_workspace_bytes(batch, k), workspace_bytes);
    }
    const bool swiglu = epilogue == JL_SWIGLU;
    // Tile: 128 x 128 when that gives most compute units a workgroup, else 64 rows x 64 columns
    // (x 128 for gate/up, whose halves must meet in one wave), which cuts a narrow projection or a
    // short batch into four (two) times as many workgroups.
    int n_tiles_128 = 0;
    for (int i = 0; i < (swiglu ? 1 : count); i++)
        n_tiles_128 += ((int)weights[i]->rows + (swiglu ? 63 : 127)) / (swiglu ? 64 : 128);
    const bool big = (int64_t)n_tiles_128 * ((rows + 127) / 128) * 2 >= (int64_t)ctx->compute_units * 3;
    const int bm = big ? 128 : 64, bn = (big || swiglu) ? 128 : 64;
    const int padded = (rows + bm - 1) / bm * bm;   // at most the 128-row padding the workspace holds

    int8_t *A8 = (int8_t *)workspace;
    const size_t a_bytes = round_up(round_up((size_t)batch, 128) * (size_t)k, 256);
    const size_t s_bytes = round_up(round_up((size_t)batch, 128) * (size_t)(k / 32) * 4, 256);
    float *dA = (float *)((uint8_t *)workspace + a_bytes);
    int32_t *sS = (int32_t *)((uint8_t *)workspace + a_bytes + s_bytes);
    const dim3 qgrid((unsigned)((k / 8 + 255) / 256), (unsigned)padded);
    if (type == JL_Q4_0)
        hipLaunchKernelGGL(jl_quantize_rows_i8<true>, qgrid, dim3(256), 0, ctx->stream, X, rows, padded, k, A8, dA, sS);
    else
        hipLaunchKernelGGL(jl_quantize_rows_i8<false>, qgrid, dim3(256), 0, ctx->stream, X, rows, padded, k, A8, dA, sS);
    JL_HIP(hipGetLastError());

    I8Params p{};
    p.A8 = A8;
    p.dA = dA;
    p.sS = sS;
    p.nseg = swiglu ? 1 : count;
    const int per_tile = swiglu ? bn / 2 : bn;
    int tiles = 0, col = 0;
    for (int i = 0; i < p.nseg; i++) {
        p.w[i] = weights[i]->blocks;
        p.seg_rows[i] = (int)weights[i]->rows;
        p.seg_tile_begin[i] = tiles;
        p.seg_col_begin[i] = col;
        tiles += ((int)weights[i]->rows + per_tile - 1) / per_tile;
        col += (int)weights[i]->rows;
    }
    p.seg_tile_begin[p.nseg] = tiles;
    p.w_up = swiglu ? weights[1]->blocks : nullptr;
    p.C = C;
    p.rows = rows;
    p.padded = padded;
    p.k = k;
    p.ldo = ldo;
    p.col_offset = col_offset;
    p.epilogue = epilogue;
    p.row_bytes = k / 32 * jl_block_bytes(type);
    p.ntiles = tiles;
    p.mtiles = padded / bm;
    return type == JL_Q8_0 ? launch_i8_tile<JL_Q8_0>(ctx, p, bm, bn) : launch_i8_tile<JL_Q4_0>(ctx, p, bm, bn);
}
