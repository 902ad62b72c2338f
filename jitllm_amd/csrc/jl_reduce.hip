// The two small reductions that sit on either side of the decode projections.
//
//   jl_rms_scale   1 / sqrt(sum x^2 / n + eps) as a device scalar -- what the reference's
//                  reductionOneBlockWithLayer leaves in slot 0 of its temp array
//                  (J/backend/tornado/kernels/TransformerComputeKernels.java:378-437) and
//                  CpuOperations.rmsnorm computes on the host (J/inference/op/CpuOperations.java:60-66);
//                  the RMS-folding projections read it.
//   jl_argmax      index of the first maximum of the logits -- argmaxLogits (:95-127) on the device,
//                  FloatTensor.argmax (J/tensor/standard/FloatTensor.java:168-181) on the host.
//
// Both are one workgroup: the inputs are a few KB to half a MB and the result is one word.
#include "jl_device.h"
#include "jl_internal.h"

#include <climits>

namespace {

constexpr int kThreads = 1024;

__global__ void __launch_bounds__(kThreads) jl_rms_scale_kernel(const float *x, int64_t n, float eps, float *scale) {
    __shared__ float part[kThreads / JL_WAVE];
    const int tid = threadIdx.x;
    float ss = 0.f;
    const int64_t n4 = ((uintptr_t)x & 15) == 0 ? n / 4 : 0;
    for (int64_t i = tid; i < n4; i += kThreads) {
        const float4 v = ((const float4 *)x)[i];
        ss = fmaf(v.x, v.x, ss);
        ss = fmaf(v.y, v.y, ss);
        ss = fmaf(v.z, v.z, ss);
        ss = fmaf(v.w, v.w, ss);
    }
    for (int64_t i = n4 * 4 + tid; i < n; i += kThreads) ss = fmaf(x[i], x[i], ss);
#pragma unroll
    for (int o = JL_WAVE / 2; o > 0; o >>= 1) ss += __shfl_xor(ss, o, JL_WAVE);
    if ((tid & (JL_WAVE - 1)) == 0) part[tid / JL_WAVE] = ss;
    __syncthreads();
    if (tid == 0) {
        float total = 0.f;
        for (int w = 0; w < kThreads / JL_WAVE; w++) total += part[w];
        // (float)(1.0 / Math.sqrt(ss / size + eps)), the division and the addition in fp32
        scale[0] = (float)(1.0 / sqrt((double)(total / (float)n + eps)));
    }
}

// larger value wins, equal values: the lower index (the first maximum of a sequential scan)
__device__ __forceinline__ void keep_better(float &v, int &i, float ov, int oi) {
    if (ov > v || (ov == v && oi < i)) {
        v = ov;
        i = oi;
    }
}

__global__ void __launch_bounds__(kThreads) jl_argmax_kernel(const float *values, int n, int32_t *index) {
    __shared__ float pv[kThreads / JL_WAVE];
    __shared__ int pi[kThreads / JL_WAVE];
    const int tid = threadIdx.x;
    float best = -INFINITY;
    int at = INT_MAX;
    const int n4 = ((uintptr_t)values & 15) == 0 ? n / 4 : 0;
    for (int i = tid; i < n4; i += kThreads) {
        const float4 v = ((const float4 *)values)[i];
        // ascending index inside a thread: a strict comparison keeps the first of equals
        if (v.x > best) { best = v.x; at = 4 * i; }
        if (v.y > best) { best = v.y; at = 4 * i + 1; }
        if (v.z > best) { best = v.z; at = 4 * i + 2; }
        if (v.w > best) { best = v.w; at = 4 * i + 3; }
    }
    for (int i = n4 * 4 + tid; i < n; i += kThreads)
        if (values[i] > best) { best = values[i]; at = i; }
#pragma unroll
    for (int o = JL_WAVE / 2; o > 0; o >>= 1) {
        const float ov = __shfl_xor(best, o, JL_WAVE);
        const int oi = __shfl_xor(at, o, JL_WAVE);
        keep_better(best, at, ov, oi);
    }
    if ((tid & (JL_WAVE - 1)) == 0) {
        pv[tid / JL_WAVE] = best;
        pi[tid / JL_WAVE] = at;
    }
    __syncthreads();
    if (tid == 0) {
        for (int w = 1; w < kThreads / JL_WAVE; w++) keep_better(best, at, pv[w], pi[w]);
        // the host scan starts from element 0 and moves only on a strictly larger value: nothing
        // beats a NaN there, and with no value above -inf it stays at 0
        if (at == INT_MAX || values[0] != values[0]) at = 0;
        index[0] = at;
    }
}

}  // namespace

int jl_launch_rms_scale(jl_context *ctx, const float *x, int64_t n, float eps, float *scale) {
    hipLaunchKernelGGL(jl_rms_scale_kernel, dim3(1), dim3(kThreads), 0, ctx->stream, x, n, eps, scale);
    JL_HIP(hipGetLastError());
    return JL_OK;
}

int jl_launch_argmax(jl_context *ctx, const float *values, int64_t n, int32_t *index) {
    hipLaunchKernelGGL(jl_argmax_kernel, dim3(1), dim3(kThreads), 0, ctx->stream, values, (int)n, index);
    JL_HIP(hipGetLastError());
    return JL_OK;
}
