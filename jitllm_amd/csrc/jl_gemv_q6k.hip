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
// One wave per weight row, sixteen lanes per super-block.  Lane (h, i) of a super-block -- half h,
// byte positions 4 i .. 4 i + 3 -- reads one dword from each ql plane and one from qh, which hold
// sixteen weights: four consecutive ones in each of the half's four groups of 32.  The 6-bit values
// are put together a dword (four weights) at a time; "- 32" and the group's scale are applied to
// the group's partial sum, not to each weight.  The weights are read straight from global memory:
// a row's bytes are used once, and the three dword streams of a wave cover whole cache lines
// between them.
#include "jl_device.h"
#include "jl_internal.h"

namespace {

struct __attribute__((packed, aligned(2))) U32a2 { uint32_t v; };
struct __attribute__((packed, aligned(2))) U64a2 { uint32_t lo, hi; };

__device__ __forceinline__ float ub(uint32_t v, int k) { return (float)((v >> (8 * k)) & 0xFFu); }

// sum over the four bytes of q (values 0..63) times x, and the sum of x
__device__ __forceinline__ void dot4(uint32_t q, const float4 x, float &qx, float &sx) {
    qx = fmaf(ub(q, 0), x.x, fmaf(ub(q, 1), x.y, fmaf(ub(q, 2), x.z, ub(q, 3) * x.w)));
    sx = (x.x + x.y) + (x.z + x.w);
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
        for (int sb = lane >> 4; sb < blocks; sb += 4) {
            const uint8_t *blk = wr + sb * 210;
            const uint32_t a = ((const U32a2 *)(blk + 64 * h + 4 * i))->v;        // ql, plane 0
            const uint32_t b = ((const U32a2 *)(blk + 64 * h + 32 + 4 * i))->v;   // ql, plane 1
            const uint32_t c = ((const U32a2 *)(blk + 128 + 32 * h + 4 * i))->v;  // qh
            const U64a2 s8 = *(const U64a2 *)(blk + 192 + 8 * h);                 // the half's 8 scales
            const float d = jl_half_bits_to_float(*(const unsigned short *)(blk + 208));
            const float4 *xs = (const float4 *)(x + sb * 256 + 128 * h + 4 * i);
            const uint32_t q0 = (a & 0x0F0F0F0Fu) | ((c & 0x03030303u) << 4);
            const uint32_t q1 = (b & 0x0F0F0F0Fu) | (((c >> 2) & 0x03030303u) << 4);
            const uint32_t q2 = ((a >> 4) & 0x0F0F0F0Fu) | (((c >> 4) & 0x03030303u) << 4);
            const uint32_t q3 = ((b >> 4) & 0x0F0F0F0Fu) | (((c >> 6) & 0x03030303u) << 4);
            // scale of group g for these positions: byte (i / 4) + 2 g of the half's eight
            const int is = i >> 2;
            const uint32_t slo = s8.lo >> (8 * is), shi = s8.hi >> (8 * is);
            const float sc0 = (float)(int)(int8_t)(slo & 0xFF), sc1 = (float)(int)(int8_t)((slo >> 16) & 0xFF);
            const float sc2 = (float)(int)(int8_t)(shi & 0xFF), sc3 = (float)(int)(int8_t)((shi >> 16) & 0xFF);
            float qx, sx;
            dot4(q0, xs[0], qx, sx);
            acc = fmaf(d * sc0, fmaf(-32.f, sx, qx), acc);
            dot4(q1, xs[8], qx, sx);
            acc = fmaf(d * sc1, fmaf(-32.f, sx, qx), acc);
            dot4(q2, xs[16], qx, sx);
            acc = fmaf(d * sc2, fmaf(-32.f, sx, qx), acc);
            dot4(q3, xs[24], qx, sx);
            acc = fmaf(d * sc3, fmaf(-32.f, sx, qx), acc);
        }
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
    hipLaunchKernelGGL(jl_gemv_q6k, dim3(groups), dim3(256), 0, ctx->stream, w->blocks, x, out, rows, n, epilogue);
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
