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
#include "jl_device.h"
#include "jl_internal.h"

namespace {

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef _Float16 half4 __attribute__((ext_vector_type(4)));
typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
typedef float floatx4 __attribute__((ext_vector_type(4)));

constexpr int kMaxWeights = 8;

// ---- activations: fp32 -> fp16 with a power-of-two row scale --------------------------------

// One wave per row: scale = the power of two that brings the row's largest magnitude into
// [2^11, 2^12); a16 = half(x / scale) (the division is exact).
__global__ void __launch_bounds__(256)
jl_rows_to_f16(const float *__restrict__ X, _Float16 *__restrict__ A, float *__restrict__ row_scale,
               int rows, int padded_rows, int k) {
    int row = blockIdx.x * 4 + threadIdx.x / JL_WAVE;
    int lane = threadIdx.x & (JL_WAVE - 1);
    if (row >= padded_rows) return;
    _Float16 *a = A + (int64_t)row * k;
    if (row >= rows) {
        for (int i = lane * 4; i < k; i += JL_WAVE * 4) *(half4 *)(a + i) = half4{0, 0, 0, 0};
        if (lane == 0) row_scale[row] = 1.f;
        return;
    }
    const float *x = X + (int64_t)row * k;
    float amax = 0.f;
    for (int i = lane * 4; i < k; i += JL_WAVE * 4) {
        float4 v = *(const float4 *)(x + i);
        amax = fmaxf(amax, fmaxf(fmaxf(fabsf(v.x), fabsf(v.y)), fmaxf(fabsf(v.z), fabsf(v.w))));
    }
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) amax = fmaxf(amax, __shfl_xor(amax, off, JL_WAVE));
    // Every row is brought to [2^11, 2^12) at its largest magnitude: huge rows stay finite in
    // fp16, tiny rows keep their bits out of fp16's subnormal range, and the power of two is
    // undone exactly in the epilogue.
    float scale = 1.f, inv = 1.f;
    if (amax > 0.f && amax < INFINITY) {
        int e;
        frexpf(amax, &e);  // amax = f * 2^e, f in [0.5, 1)
        e = e < -100 ? -100 : e;
        scale = ldexpf(1.f, e - 12);
        inv = ldexpf(1.f, 12 - e);
    }
    for (int i = lane * 4; i < k; i += JL_WAVE * 4) {
        float4 v = *(const float4 *)(x + i);
        half4 h = {(_Float16)(v.x * inv), (_Float16)(v.y * inv), (_Float16)(v.z * inv),
                   (_Float16)(v.w * inv)};
        *(half4 *)(a + i) = h;
    }
    if (lane == 0) row_scale[row] = scale;
}

// ---- weight slice decode: 32 consecutive elements of one row -> fp16 -------------------------

// `blk` addresses the 32-element unit: a Q8_0 / Q4_0 block, or for Q4_K the super-block with
// `sub` naming the 32-element sub-block.  Each value is the host decode rounded once to fp16.
template <int TYPE>
__device__ __forceinline__ void decode32_to_f16(const uint8_t *blk, int sub, _Float16 *dst) {
    if constexpr (TYPE == JL_Q8_0) {
        // 34 bytes, 2-byte aligned: read as 17 halfwords
        const uint16_t *h = (const uint16_t *)blk;
        float d = jl_half_bits_to_float(h[0]);
#pragma unroll
        for (int i = 0; i < 16; i++) {
            uint32_t v = h[1 + i];
            float q0 = (float)(int)(int8_t)(v & 0xFF);
            float q1 = (float)(int)(int8_t)(v >> 8);
            dst[2 * i] = (_Float16)__fmul_rn(q0, d);
            dst[2 * i + 1] = (_Float16)__fmul_rn(q1, d);
        }
    } else if constexpr (TYPE == JL_Q4_0) {
        const uint16_t *h = (const uint16_t *)blk;
        float d = jl_half_bits_to_float(h[0]);
#pragma unroll
        for (int i = 0; i < 8; i++) {
            uint32_t v = h[1 + i];  // bytes 2i, 2i+1
            dst[2 * i] = (_Float16)__fmul_rn((float)((int)(v & 0xF) - 8), d);
            dst[2 * i + 1] = (_Float16)__fmul_rn((float)((int)((v >> 8) & 0xF) - 8), d);
            dst[16 + 2 * i] = (_Float16)__fmul_rn((float)((int)((v >> 4) & 0xF) - 8), d);
            dst[16 + 2 * i + 1] = (_Float16)__fmul_rn((float)((int)(v >> 12) - 8), d);
        }
    } else {
        const uint32_t *hdr = (const uint32_t *)blk;
        uint32_t h0 = hdr[0];
        float d = jl_half_bits_to_float(h0);
        float dmin = jl_half_bits_to_float(h0 >> 16);
        int sc, mn;
        jl_q4k_scale_min(hdr[1], hdr[2], hdr[3], sub, sc, mn);
        float ds = __fmul_rn(d, (float)sc);
        float dm = __fmul_rn(dmin, (float)mn);
        const uint32_t *qs = (const uint32_t *)(blk + 16 + (sub >> 1) * 32);
        int shift = (sub & 1) * 4;
#pragma unroll
        for (int i = 0; i < 8; i++) {
            uint32_t v = (qs[i] >> shift) & 0x0F0F0F0Fu;
#pragma unroll
            for (int b = 0; b < 4; b++) {
                float q = (float)((v >> (8 * b)) & 0xFF);
                dst[4 * i + b] = (_Float16)__fsub_rn(__fmul_rn(ds, q), dm);
            }
        }
    }
}

struct GemmParams {
    const uint8_t *w[kMaxWeights];
    int w_rows[kMaxWeights];
    int w_begin[kMaxWeights + 1];  // first virtual output column of each weight
    int count;
    const _Float16 *A;       // [padded_rows x k] fp16
    const float *row_scale;  // [padded_rows]
    float *C;
    int rows;                // active rows
    int k;
    int n_total;             // virtual output columns (SWIGLU: rows of one weight)
    int64_t ldo;
    int64_t col_offset;
    int epilogue;
    int row_bytes;
};

constexpr int BM = 128, BN = 128, BK = 64;
constexpr int LDS_STRIDE = BK + 8;  // halfs; 144-byte rows keep 16-byte fragment reads conflict-light

// Workgroup: 256 threads = 4 waves as 2 (M) x 2 (N); wave tile 64 x 64 = 4 x 4 MFMA blocks of
// 16 x 16.  For JL_SWIGLU the 128 tile columns are 64 gate rows followed by the 64 up rows of the
// same output columns, and a wave's four column blocks are {gate, gate, up, up} of its 32 outputs.
template <int TYPE>
__global__ void __launch_bounds__(256) jl_gemm_f16(GemmParams p) {
    __shared__ __attribute__((aligned(16))) _Float16 As[2][BM * LDS_STRIDE];
    __shared__ __attribute__((aligned(16))) _Float16 Ws[2][BN * LDS_STRIDE];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;
    const int m0 = blockIdx.y * BM;
    const bool swiglu = p.epilogue == JL_SWIGLU;
    const int cols_per_tile = swiglu ? BN / 2 : BN;
    const int n0 = blockIdx.x * cols_per_tile;  // first virtual output column of the tile

    // --- loader roles ---
    // weights: thread t decodes 32 elements: tile row t / 2, half (t & 1) of the 64-wide slice
    const int wr = tid >> 1;
    const int wh = tid & 1;
    const uint8_t *wrow = nullptr;  // start of the source weight row, or null past the last column
    {
        int vcol;
        int widx = 0;
        if (swiglu) {
            widx = wr >= 64 ? 1 : 0;
            vcol = n0 + (wr & 63);
            if (vcol < p.n_total) wrow = p.w[widx] + (int64_t)vcol * p.row_bytes;
        } else {
            vcol = n0 + wr;
            if (vcol < p.n_total) {
#pragma unroll
                for (int i = 1; i < kMaxWeights; i++)
                    if (i < p.count && vcol >= p.w_begin[i]) widx = i;
                wrow = p.w[widx] + (int64_t)(vcol - p.w_begin[widx]) * p.row_bytes;
            }
        }
    }
    // activations: thread t copies 32 halfs (64 bytes): tile row t / 2, half (t & 1)
    const _Float16 *arow = p.A + (int64_t)(m0 + (tid >> 1)) * p.k + (tid & 1) * 32;

    half8 a_stage[4];
    _Float16 w_stage[32];

    auto load = [&](int kt) {
        const half8 *src = (const half8 *)(arow + kt * BK);
#pragma unroll
        for (int i = 0; i < 4; i++) a_stage[i] = src[i];
        if (wrow) {
            if constexpr (TYPE == JL_Q4_K) {
                int e = kt * BK + wh * 32;  // element index in the row
                decode32_to_f16<TYPE>(wrow + (e >> 8) * 144, (e & 255) >> 5, w_stage);
            } else {
                constexpr int BB = TYPE == JL_Q8_0 ? 34 : 18;
                decode32_to_f16<TYPE>(wrow + (int64_t)(kt * 2 + wh) * BB, 0, w_stage);
            }
        } else {
#pragma unroll
            for (int i = 0; i < 32; i++) w_stage[i] = (_Float16)0;
        }
    };
    auto commit = [&](int buf) {
        half8 *ad = (half8 *)(&As[buf][(tid >> 1) * LDS_STRIDE + (tid & 1) * 32]);
#pragma unroll
        for (int i = 0; i < 4; i++) ad[i] = a_stage[i];
        half8 *wd = (half8 *)(&Ws[buf][wr * LDS_STRIDE + wh * 32]);
#pragma unroll
        for (int i = 0; i < 4; i++) {
            half8 v;
#pragma unroll
            for (int j = 0; j < 8; j++) v[j] = w_stage[8 * i + j];
            wd[i] = v;
        }
    };

    floatx4 acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; i++)
#pragma unroll
        for (int j = 0; j < 4; j++) acc[i][j] = floatx4{0.f, 0.f, 0.f, 0.f};

    // LDS row of each of the wave's four column blocks
    int brow[4];
#pragma unroll
    for (int j = 0; j < 4; j++) {
        if (swiglu) brow[j] = (j >> 1) * 64 + wn * 32 + (j & 1) * 16;
        else brow[j] = wn * 64 + j * 16;
    }

    const int ksteps = p.k / BK;
    load(0);
    for (int kt = 0; kt < ksteps; kt++) {
        const int buf = kt & 1;
        commit(buf);
        __syncthreads();
        if (kt + 1 < ksteps) load(kt + 1);
#pragma unroll
        for (int ks = 0; ks < BK / 32; ks++) {
            half8 a[4], b[4];
            const int koff = ks * 32 + (lane >> 4) * 8;
#pragma unroll
            for (int i = 0; i < 4; i++)
                a[i] = *(const half8 *)(&As[buf][(wm * 64 + i * 16 + (lane & 15)) * LDS_STRIDE + koff]);
#pragma unroll
            for (int j = 0; j < 4; j++)
                b[j] = *(const half8 *)(&Ws[buf][(brow[j] + (lane & 15)) * LDS_STRIDE + koff]);
#pragma unroll
            for (int i = 0; i < 4; i++)
#pragma unroll
                for (int j = 0; j < 4; j++)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a[i], b[j], acc[i][j], 0, 0, 0);
        }
    }

    // epilogue: lane holds rows 4 * (lane / 16) + e, column lane % 16 of each 16 x 16 block
#pragma unroll
    for (int i = 0; i < 4; i++) {
#pragma unroll
        for (int e = 0; e < 4; e++) {
            int m = m0 + wm * 64 + i * 16 + (lane >> 4) * 4 + e;
            if (m >= p.rows) continue;
            float rs = p.row_scale[m];
            float *crow = p.C + (int64_t)m * p.ldo + p.col_offset;
            if (swiglu) {
#pragma unroll
                for (int j = 0; j < 2; j++) {
                    int col = n0 + wn * 32 + j * 16 + (lane & 15);
                    if (col < p.n_total)
                        crow[col] = jl_swiglu_value(acc[i][j][e] * rs, acc[i][j + 2][e] * rs);
                }
            } else {
#pragma unroll
                for (int j = 0; j < 4; j++) {
                    int col = n0 + wn * 64 + j * 16 + (lane & 15);
                    if (col < p.n_total) {
                        float v = acc[i][j][e] * rs;
                        if (p.epilogue == JL_RESIDUAL) crow[col] += v;
                        else crow[col] = v;
                    }
                }
            }
        }
    }
}

size_t round_up(size_t v, size_t a) { return (v + a - 1) / a * a; }

}  // namespace

size_t jl_gemm_workspace_bytes_impl(int64_t max_rows, int64_t cols, int math) {
    size_t padded = round_up((size_t)max_rows, BM);
    if (math == JL_MATH_INT8) {
        return round_up(padded * (size_t)cols, 256) + round_up(padded * (size_t)(cols / 32) * 4, 256);
    }
    return round_up(padded * (size_t)cols * 2, 256) + round_up(padded * 4, 256);
}

int jl_launch_gemm(jl_context *ctx, const jl_weight *const *weights, int count, const float *X,
                   float *C, int64_t batch, int64_t active_rows, int64_t ldo, int64_t col_offset,
                   int epilogue, int math, void *workspace, size_t workspace_bytes) {
    (void)workspace_bytes;
    const int type = weights[0]->type;
    const int k = (int)weights[0]->cols;
    if (math == JL_MATH_INT8) {
        return jl_fail(JL_ERR_UNSUPPORTED, "jl_gemm: the int8 kernels are not built into this library");
    }
    JL_REQUIRE(k % 64 == 0, "jl_gemm: row length %d is not a multiple of 64", k);
    JL_REQUIRE(((uintptr_t)X & 15) == 0 && ((uintptr_t)workspace & 255) == 0,
               "jl_gemm: X must be 16-byte and the workspace 256-byte aligned");
    const int rows = (int)active_rows;
    const int padded = (int)round_up((size_t)rows, BM);
    // the workspace was sized for `batch` rows, of which `rows` <= batch are converted
    _Float16 *A = (_Float16 *)workspace;
    float *row_scale =
        (float *)((uint8_t *)workspace + round_up(round_up((size_t)batch, BM) * (size_t)k * 2, 256));

    hipLaunchKernelGGL(jl_rows_to_f16, dim3((padded + 3) / 4), dim3(256), 0, ctx->stream, X, A,
                       row_scale, rows, padded, k);
    JL_HIP(hipGetLastError());

    GemmParams p{};
    p.count = count;
    int begin = 0;
    for (int i = 0; i < count; i++) {
        p.w[i] = weights[i]->blocks;
        p.w_rows[i] = (int)weights[i]->rows;
        p.w_begin[i] = begin;
        begin += (int)weights[i]->rows;
    }
    p.w_begin[count] = begin;
    p.A = A;
    p.row_scale = row_scale;
    p.C = C;
    p.rows = rows;
    p.k = k;
    p.n_total = epilogue == JL_SWIGLU ? (int)weights[0]->rows : begin;
    p.ldo = ldo;
    p.col_offset = col_offset;
    p.epilogue = epilogue;
    p.row_bytes = k / jl_block_elems(type) * jl_block_bytes(type);

    const int cols_per_tile = epilogue == JL_SWIGLU ? BN / 2 : BN;
    dim3 grid((p.n_total + cols_per_tile - 1) / cols_per_tile, padded / BM);
    switch (type) {
        case JL_Q8_0:
            hipLaunchKernelGGL(jl_gemm_f16<JL_Q8_0>, grid, dim3(256), 0, ctx->stream, p);
            break;
        case JL_Q4_0:
            hipLaunchKernelGGL(jl_gemm_f16<JL_Q4_0>, grid, dim3(256), 0, ctx->stream, p);
            break;
        case JL_Q4_K:
            hipLaunchKernelGGL(jl_gemm_f16<JL_Q4_K>, grid, dim3(256), 0, ctx->stream, p);
            break;
        default:
            return jl_fail(JL_ERR_UNSUPPORTED, "jl_gemm: no kernel for a ggml type %d weight", type);
    }
    JL_HIP(hipGetLastError());
    return JL_OK;
}
