// Single-token projection over a Q6_K weight: out (+)= W . x.
//
// Files quantised "Q4_K_M" keep their vocabulary projection and some attention / feed-forward
// tensors in Q6_K, and the reference reads a projection "by its own representation, not the plan's"
// (J/backend/tornado/layers/type/q8_0/LogitsQ8_0Layer.java:92-96), so a Q4_K model needs this
// kernel beside the Q4_K ones.  Replaces matrixVectorGenericQ6_K / ...WithResidualQ6_K
// (J/backend/tornado/kernels/TransformerComputeKernelsQ6_K.java:548-590); the arithmetic is
// Q6_KFloatTensor's (J/tensor/standard/Q6_KFloatTensor.java:66-122): a super-block of 256 weights
// is ql[128] | qh[64] | 16 signed scales | fp16 d, w = d * scale * (q - 32).
//
// One wave per weight row, sixteen lanes per super-block.  A lane reads eight consecutive ql bytes
// and the eight qh bytes of the same positions, which hold sixteen weights: eight consecutive ones
// in each of two of the half's four groups of 32.  The 6-bit values are put together a dword (four
// weights) at a time; "- 32" and the group's scale are applied to the group's partial sum, not to
// each weight.  The weights are read straight from global memory (a row's bytes are used once):
// the sixteen lanes of a super-block read its ql as one contiguous 128-byte run.  For the usual
// row lengths a lane's activations are the same in every row and stay in registers.
#include "jl_device.h"
#include "jl_internal.h"

namespace {

struct __attribute__((packed, aligned(2))) U32a2 { uint32_t v; };
struct __attribute__((packed, aligned(2))) U64a2 { uint32_t lo, hi; };

__device__ __forceinline__ float ub(uint32_t v, int k) { return (float)((v >> (8 * k)) & 0xFFu); }

// sum over the four bytes of q (values 0..63) times x
__device__ __forceinline__ float dot4(uint32_t q, const float4 x) {
    return fmaf(ub(q, 0), x.x, fmaf(ub(q, 1), x.y, fmaf(ub(q, 2), x.z, ub(q, 3) * x.w)));
}

// What lane (h, i) reads of one super-block: eight consecutive ql bytes -- lanes i < 4 of plane 0
// (groups 0 and 2 of the half), lanes i >= 4 of plane 1 (groups 1 and 3) -- so that the sixteen
// lanes of a super-block read its ql in one contiguous 128-byte run, and the eight qh bytes of
// the same positions.
struct Raw {
    U64a2 ql, qh;
    U64a2 s8;              // the half's 8 scales
    unsigned short d;
};
// The sixteen activations that go with it: eight consecutive ones of the low-nibble group and
// eight of the high-nibble group, with -32 times their sums (the "- 32" of every weight, applied
// to the group's sum).
struct Xs {
    float4 x[4];
    float m32[2];
};

__device__ __forceinline__ Raw load_raw(const uint8_t *blk, int h, int i) {
    Raw r;
    r.ql = *(const U64a2 *)(blk + 64 * h + 32 * (i >> 2) + 8 * (i & 3));
    r.qh = *(const U64a2 *)(blk + 128 + 32 * h + 8 * (i & 3));
    r.s8 = *(const U64a2 *)(blk + 192 + 8 * h);
    r.d = *(const unsigned short *)(blk + 208);
    return r;
}

__device__ __forceinline__ Xs load_x(const float *x, int h, int i) {
    Xs v;
    const float4 *xs = (const float4 *)(x + 128 * h + 32 * (i >> 2) + 8 * (i & 3));
    v.x[0] = xs[0];
    v.x[1] = xs[1];
    v.x[2] = xs[16];   // 64 elements on: the high-nibble group
    v.x[3] = xs[17];
#pragma unroll
    for (int g = 0; g < 2; g++) {
        const float4 p = v.x[2 * g], q = v.x[2 * g + 1];
        v.m32[g] = -32.f * (((p.x + p.y) + (p.z + p.w)) + ((q.x + q.y) + (q.z + q.w)));
    }
    return v;
}

__device__ __forceinline__ float block_part(const Raw &r, const Xs &v, int i) {
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
}

__global__ void __launch_bounds__(256)
jl_gemv_q6k(const uint8_t *__restrict__ w, const float *__restrict__ x, float *__restrict__ out, int rows,
            int n, int epilogue) {
    const int lane = threadIdx.x & 63;
    const int waves = (gridDim.x * blockDim.x) >> 6;
    const int blocks = n >> 8;                 // super-blocks per row
    const int j = lane & 15, h = j >> 3, i = j & 7;
    for (int row = (blockIdx.x * blockDim.x + threadIdx.x) >> 6; row < rows; row += waves) {
        const uint8_t *wr = w + (int64_t)row * blocks * 210;
        float acc = 0.f;
        // two super-blocks per lane and trip: all their loads are issued before the first use, which
        // doubles the bytes each wave keeps in flight (short rows are otherwise latency-bound)
        for (int sb0 = lane >> 4; sb0 < blocks; sb0 += 8) {
            Raw r[2];
            Xs v[2];
#pragma unroll
            for (int u = 0; u < 2; u++) {
                const int sb = sb0 + 4 * u;
                if (sb < blocks) {
                    r[u] = load_raw(wr + sb * 210, h, i);
                    v[u] = load_x(x + sb * 256, h, i);
                }
            }
#pragma unroll
            for (int u = 0; u < 2; u++)
                if (sb0 + 4 * u < blocks) acc += block_part(r[u], v[u], i);
        }
        acc = jl_group_sum<JL_WAVE>(acc);
        if (lane == 0) {
            if (epilogue == JL_RESIDUAL) out[row] += acc;
            else out[row] = acc;
        }
    }
}

// Rows of 4 NIT super-blocks: a lane meets the same activations in every row, so they are read
// once into registers, and a row's 6 NIT loads per lane are all in flight before the first use.
template <int NIT>
__global__ void __launch_bounds__(256)
jl_gemv_q6k_held(const uint8_t *__restrict__ w, const float *__restrict__ x, float *__restrict__ out, int rows,
                 int epilogue) {
    const int lane = threadIdx.x & 63;
    const int waves = (gridDim.x * blockDim.x) >> 6;
    const int j = lane & 15, h = j >> 3, i = j & 7;
    Xs v[NIT];
#pragma unroll
    for (int k = 0; k < NIT; k++) v[k] = load_x(x + ((lane >> 4) + 4 * k) * 256, h, i);
    for (int row = (blockIdx.x * blockDim.x + threadIdx.x) >> 6; row < rows; row += waves) {
        const uint8_t *wr = w + (int64_t)row * (4 * NIT * 210) + (lane >> 4) * 210;
        Raw r[NIT];
#pragma unroll
        for (int k = 0; k < NIT; k++) r[k] = load_raw(wr + k * 840, h, i);
        float acc = 0.f;
#pragma unroll
        for (int k = 0; k < NIT; k++) acc += block_part(r[k], v[k], i);
        acc = jl_group_sum<JL_WAVE>(acc);
        if (lane == 0) {
            if (epilogue == JL_RESIDUAL) out[row] += acc;
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
    out[e] = __fmul_rn(__fmul_rn(d, (float)sc), (float)q);
}

}  // namespace

int jl_launch_gemv_q6k(jl_context *ctx, const jl_weight *w, const float *x, float *out, int epilogue) {
    const int rows = (int)w->rows, n = (int)w->cols;
    if (n % 256 != 0 || ((uintptr_t)x & 15) != 0) {
        return jl_fail(JL_ERR_UNSUPPORTED,
                       "no Q6_K projection kernel for a row length of %d or an unaligned vector", n);
    }
    // enough waves to hide the loads' latency, rows dealt round robin
    int groups = (rows + 3) / 4;
    const int cap = ctx->compute_units * 8;
    if (groups > cap) groups = cap;
    switch (n) {
        case 1024:
            hipLaunchKernelGGL(jl_gemv_q6k_held<1>, dim3(groups), dim3(256), 0, ctx->stream, w->blocks, x, out, rows, epilogue);
            break;
        case 2048:
            hipLaunchKernelGGL(jl_gemv_q6k_held<2>, dim3(groups), dim3(256), 0, ctx->stream, w->blocks, x, out, rows, epilogue);
            break;
        case 4096:
            hipLaunchKernelGGL(jl_gemv_q6k_held<4>, dim3(groups), dim3(256), 0, ctx->stream, w->blocks, x, out, rows, epilogue);
            break;
        case 8192:
            hipLaunchKernelGGL(jl_gemv_q6k_held<8>, dim3(groups), dim3(256), 0, ctx->stream, w->blocks, x, out, rows, epilogue);
            break;
        default:
            hipLaunchKernelGGL(jl_gemv_q6k, dim3(groups), dim3(256), 0, ctx->stream, w->blocks, x, out, rows, n, epilogue);
            break;
    }
    JL_HIP(hipGetLastError());
    return JL_OK;
}

int jl_launch_dequant_q6k(jl_context *ctx, const jl_weight *w, float *out) {
    const int64_t total = w->rows * w->cols;
    hipLaunchKernelGGL(jl_dequant_q6_k, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, ctx->stream, w->blocks,
                       out, total);
    JL_HIP(hipGetLastError());
    return JL_OK;
}
