// Element-wise decode of GGUF blocks to fp32 with the host tensors' own arithmetic, plus the small
// element-wise kernels (fill, SwiGLU).  The decode kernels exist so the weight arithmetic can be
// held bit-equal to Q8_0FloatTensor.getFloat / Q4_0FloatTensor.getFloat / Q4_KFloatTensor.getFloat.
#include "jl_device.h"
#include "jl_internal.h"

// One thread per element; every product is a separately rounded fp32 operation (jl_mul_rn: the
// compiler would otherwise contract a*b-c into one fma, which Java never does).

// J/tensor/standard/Q8_0FloatTensor.java:52-61: quant * scale.
__global__ void __launch_bounds__(256)
jl_dequant_q8_0(const uint8_t *__restrict__ w, float *__restrict__ out, int64_t total) {
    int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= total) return;
    const uint8_t *blk = w + (i >> 5) * 34;
    float d = jl_half_bits_to_float(blk[0] | (blk[1] << 8));
    float q = (float)(int)(int8_t)blk[2 + (i & 31)];
    out[i] = jl_mul_rn(q, d);
}

// J/tensor/standard/Q4_0FloatTensor.java:55-79: (nibble - 8) * scale; element i < 16 is the low
// nibble of byte i, element i >= 16 the high nibble of byte i - 16.
__global__ void __launch_bounds__(256)
jl_dequant_q4_0(const uint8_t *__restrict__ w, float *__restrict__ out, int64_t total) {
    int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= total) return;
    const uint8_t *blk = w + (i >> 5) * 18;
    float d = jl_half_bits_to_float(blk[0] | (blk[1] << 8));
    int e = (int)(i & 31);
    int byte = blk[2 + (e & 15)];
    int q = (e < 16 ? (byte & 0xF) : (byte >> 4)) - 8;
    out[i] = jl_mul_rn((float)q, d);
}

// J/tensor/standard/Q4_KFloatTensor.java:87-122: ((d * sc) * q) - (dmin * m).
__global__ void __launch_bounds__(256)
jl_dequant_q4_k(const uint8_t *__restrict__ w, float *__restrict__ out, int64_t total) {
    int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= total) return;
    const uint8_t *blk = w + (i >> 8) * 144;
    const uint32_t *hdr = (const uint32_t *)blk;  // super-blocks are 16-byte aligned
    uint32_t h0 = hdr[0];
    float d = jl_half_bits_to_float(h0);
    float dmin = jl_half_bits_to_float(h0 >> 16);
    int within = (int)(i & 255);
    int pair = within >> 6;
    int pos = within & 63;
    int high = pos >> 5;
    int byte = blk[16 + pair * 32 + (pos & 31)];
    int q = high ? (byte >> 4) : (byte & 0xF);
    int sc, mn;
    jl_q4k_scale_min(hdr[1], hdr[2], hdr[3], pair * 2 + high, sc, mn);
    float t = jl_mul_rn(d, (float)sc);
    t = jl_mul_rn(t, (float)q);
    float u = jl_mul_rn(dmin, (float)mn);
    out[i] = __fsub_rn(t, u);
}

__global__ void __launch_bounds__(256)
jl_fill_kernel(float *__restrict__ dst, float value, size_t count) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < count) dst[i] = value;
}

__global__ void __launch_bounds__(256)
jl_swiglu_kernel(float *__restrict__ gate, const float *__restrict__ up, int64_t count) {
    int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < count) gate[i] = jl_swiglu_value(gate[i], up[i]);
}

// batchedResidualAddFP32 (J/backend/tornado/kernels/TransformerBatchPrefillKernels.java:1078-1084):
// residual[i] = residual[i] + delta[i].
__global__ void __launch_bounds__(256)
jl_residual_add_kernel(float *__restrict__ residual, const float *__restrict__ delta, int64_t count) {
    int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < count) residual[i] = __fadd_rn(residual[i], delta[i]);
}

int jl_launch_dequant(jl_context *ctx, const jl_weight *w, float *out) {
    int64_t total = w->rows * w->cols;
    unsigned grid = (unsigned)((total + 255) / 256);
    switch (w->type) {
        case JL_Q8_0:
            hipLaunchKernelGGL(jl_dequant_q8_0, dim3(grid), dim3(256), 0, ctx->stream, w->blocks, out,
                               total);
            break;
        case JL_Q4_0:
            hipLaunchKernelGGL(jl_dequant_q4_0, dim3(grid), dim3(256), 0, ctx->stream, w->blocks, out,
                               total);
            break;
        case JL_Q4_K:
            hipLaunchKernelGGL(jl_dequant_q4_k, dim3(grid), dim3(256), 0, ctx->stream, w->blocks, out,
                               total);
            break;
        case JL_Q6_K:
        case JL_Q5_K:
        case JL_Q4_1:
        case JL_Q5_0:
        case JL_IQ4_XS:
            return jl_launch_dequant_direct(ctx, w, out);
        default:
            return jl_fail(JL_ERR_UNSUPPORTED, "jl_dequant_f32: no decode kernel for ggml type %d",
                           w->type);
    }
    JL_HIP(hipGetLastError());
    return JL_OK;
}

int jl_launch_fill(jl_context *ctx, float *dst, float value, size_t count) {
    unsigned grid = (unsigned)((count + 255) / 256);
    hipLaunchKernelGGL(jl_fill_kernel, dim3(grid), dim3(256), 0, ctx->stream, dst, value, count);
    JL_HIP(hipGetLastError());
    return JL_OK;
}

int jl_launch_swiglu(jl_context *ctx, float *gate, const float *up, int64_t count) {
    unsigned grid = (unsigned)((count + 255) / 256);
    hipLaunchKernelGGL(jl_swiglu_kernel, dim3(grid), dim3(256), 0, ctx->stream, gate, up, count);
    JL_HIP(hipGetLastError());
    return JL_OK;
}

int jl_launch_residual_add(jl_context *ctx, float *residual, const float *delta, int64_t count) {
    unsigned grid = (unsigned)((count + 255) / 256);
    hipLaunchKernelGGL(jl_residual_add_kernel, dim3(grid), dim3(256), 0, ctx->stream, residual, delta, count);
    JL_HIP(hipGetLastError());
    return JL_OK;
}
