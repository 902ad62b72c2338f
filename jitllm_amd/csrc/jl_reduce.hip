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
//   jl_quantize_q8 the activation as Q8 blocks for the packed-integer projections -- 32 signed bytes,
//                  an fp32 scale and the sum of the bytes per block: quantizeActivationQ8Blocks
//                  (J/backend/tornado/kernels/TransformerComputeKernelsQ4_0.java:287-341).
//
//   jl_rms_apply_xf16  the batched prefill's normalisation, which hands the projections fp16 rows:
//                  batchedRmsReduceParallel + batchedRmsApplyFP16
//                  (J/backend/tornado/kernels/TransformerBatchPrefillKernels.java:1480-1510, 59-72).
//
// jl_rms_scale is one workgroup (a few KB of input); jl_argmax spreads the half MB of logits over
// up to 128 workgroups and folds their results in a second, single-workgroup launch.
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

// Two launches: workgroup g scans the float4s g, g + G, ... and leaves its best (value, index) in
// the context's scratch; one small workgroup then folds the G cells.  (A single launch whose last
// workgroup folds needs device-scope fences, which cost more here than the second launch.)
constexpr int kArgmaxGroups = 128, kArgmaxThreads = 256;

struct ArgmaxCells {
    float value[kArgmaxGroups];
    int index[kArgmaxGroups];
};

__device__ __forceinline__ void fold_waves(float &best, int &at, float *pv, int *pi, int tid, int waves) {
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
    if (tid == 0)
        for (int w = 1; w < waves; w++) keep_better(best, at, pv[w], pi[w]);
}

__global__ void __launch_bounds__(kArgmaxThreads) jl_argmax_scan(const float *values, int n, ArgmaxCells *cells) {
    __shared__ float pv[kArgmaxThreads / JL_WAVE];
    __shared__ int pi[kArgmaxThreads / JL_WAVE];
    const int tid = threadIdx.x;
    float best = -INFINITY;
    int at = INT_MAX;
    const int n4 = ((uintptr_t)values & 15) == 0 ? n / 4 : 0;
    for (int i = blockIdx.x * kArgmaxThreads + tid; i < n4; i += gridDim.x * kArgmaxThreads) {
        const float4 v = ((const float4 *)values)[i];
        // ascending index inside a thread: a strict comparison keeps the first of equals
        if (v.x > best) { best = v.x; at = 4 * i; }
        if (v.y > best) { best = v.y; at = 4 * i + 1; }
        if (v.z > best) { best = v.z; at = 4 * i + 2; }
        if (v.w > best) { best = v.w; at = 4 * i + 3; }
    }
    for (int i = n4 * 4 + blockIdx.x * kArgmaxThreads + tid; i < n; i += gridDim.x * kArgmaxThreads)
        if (values[i] > best) { best = values[i]; at = i; }
    fold_waves(best, at, pv, pi, tid, kArgmaxThreads / JL_WAVE);
    if (tid == 0) {
        cells->value[blockIdx.x] = best;
        cells->index[blockIdx.x] = at;
    }
}

__global__ void __launch_bounds__(kArgmaxGroups) jl_argmax_fold(const float *values, const ArgmaxCells *cells,
                                                                int groups, int32_t *index) {
    __shared__ float pv[kArgmaxGroups / JL_WAVE];
    __shared__ int pi[kArgmaxGroups / JL_WAVE];
    const int tid = threadIdx.x;
    float best = tid < groups ? cells->value[tid] : -INFINITY;
    int at = tid < groups ? cells->index[tid] : INT_MAX;
    fold_waves(best, at, pv, pi, tid, kArgmaxGroups / JL_WAVE);
    if (tid == 0) {
        // the host scan starts from element 0 and moves only on a strictly larger value: nothing
        // beats a NaN there, and with no value above -inf it stays at 0
        if (at == INT_MAX || values[0] != values[0]) at = 0;
        index[0] = at;
    }
}

// Per-row argmax over batched logits, one workgroup per row: batchedArgmaxLogits
// (J/backend/tornado/kernels/TransformerBatchPrefillKernels.java:2118-2159), the last task of the
// reference's batched logits graph (J/backend/tornado/batch/TornadoBatchExecutor.java:226-232), with
// the host scan's rule for equal maxima -- the first one, FloatTensor.argmax -- where the reference
// kernel's tree keeps whichever its lower thread held.
__global__ void __launch_bounds__(kThreads) jl_argmax_rows_kernel(const float *values, int n, int64_t row_stride,
                                                                  int32_t *indices) {
    __shared__ float pv[kThreads / JL_WAVE];
    __shared__ int pi[kThreads / JL_WAVE];
    const int tid = threadIdx.x;
    const float *row = values + (int64_t)blockIdx.x * row_stride;
    float best = -INFINITY;
    int at = INT_MAX;
    const int n4 = ((uintptr_t)row & 15) == 0 ? n / 4 : 0;
    for (int i = tid; i < n4; i += kThreads) {
        const float4 v = ((const float4 *)row)[i];
        if (v.x > best) { best = v.x; at = 4 * i; }
        if (v.y > best) { best = v.y; at = 4 * i + 1; }
        if (v.z > best) { best = v.z; at = 4 * i + 2; }
        if (v.w > best) { best = v.w; at = 4 * i + 3; }
    }
    for (int i = n4 * 4 + tid; i < n; i += kThreads)
        if (row[i] > best) { best = row[i]; at = i; }
    fold_waves(best, at, pv, pi, tid, kThreads / JL_WAVE);
    if (tid == 0) {
        if (at == INT_MAX || row[0] != row[0]) at = 0;   // as in jl_argmax_fold
        indices[blockIdx.x] = at;
    }
}

// The same with each row cut into `chunks` runs, one workgroup per (run, row), for batches too small
// to fill the chip with a workgroup per row: the runs' best (value, index) go to cells
// [row * chunks + run] and jl_argmax_rows_fold, one wave per row, folds them.
__global__ void __launch_bounds__(kArgmaxThreads) jl_argmax_rows_scan(const float *values, int n, int64_t row_stride, int chunks,
                                                                      float *cell_value, int *cell_index) {
    __shared__ float pv[kArgmaxThreads / JL_WAVE];
    __shared__ int pi[kArgmaxThreads / JL_WAVE];
    const int tid = threadIdx.x, run = blockIdx.x;
    const float *row = values + (int64_t)blockIdx.y * row_stride;
    float best = -INFINITY;
    int at = INT_MAX;
    const int n4 = ((uintptr_t)row & 15) == 0 ? n / 4 : 0;
    const int per4 = (n4 + chunks - 1) / chunks;
    const int end4 = (run + 1) * per4 < n4 ? (run + 1) * per4 : n4;
    for (int i = run * per4 + tid; i < end4; i += kArgmaxThreads) {
        const float4 v = ((const float4 *)row)[i];
        if (v.x > best) { best = v.x; at = 4 * i; }
        if (v.y > best) { best = v.y; at = 4 * i + 1; }
        if (v.z > best) { best = v.z; at = 4 * i + 2; }
        if (v.w > best) { best = v.w; at = 4 * i + 3; }
    }
    // what the 16-byte loads do not cover (the last values of a row, or all of a row that starts off
    // a 16-byte boundary), shared out over the runs the same way
    const int rest = n - 4 * n4, per = (rest + chunks - 1) / chunks;
    const int end = (run + 1) * per < rest ? (run + 1) * per : rest;
    for (int i = run * per + tid; i < end; i += kArgmaxThreads)
        if (row[4 * n4 + i] > best) { best = row[4 * n4 + i]; at = 4 * n4 + i; }
    fold_waves(best, at, pv, pi, tid, kArgmaxThreads / JL_WAVE);
    if (tid == 0) {
        cell_value[blockIdx.y * chunks + run] = best;
        cell_index[blockIdx.y * chunks + run] = at;
    }
}

__global__ void __launch_bounds__(JL_WAVE) jl_argmax_rows_fold(const float *values, int64_t row_stride, int chunks,
                                                               const float *cell_value, const int *cell_index,
                                                               int32_t *indices) {
    const int lane = threadIdx.x, row = blockIdx.x;
    float best = lane < chunks ? cell_value[row * chunks + lane] : -INFINITY;
    int at = lane < chunks ? cell_index[row * chunks + lane] : INT_MAX;
#pragma unroll
    for (int o = JL_WAVE / 2; o > 0; o >>= 1) {
        const float ov = __shfl_xor(best, o, JL_WAVE);
        const int oi = __shfl_xor(at, o, JL_WAVE);
        keep_better(best, at, ov, oi);
    }
    if (lane == 0) {
        const float first = values[(int64_t)row * row_stride];
        if (at == INT_MAX || first != first) at = 0;   // as in jl_argmax_fold
        indices[row] = at;
    }
}

// The fold for cells a projection kernel left (one per workgroup, up to a thousand, rows in no
// particular order from cell to cell): the same rule, a strided walk first.
constexpr int kProjectionCells = JL_CONTEXT_SCRATCH_BYTES / 8;
__global__ void __launch_bounds__(kArgmaxThreads) jl_argmax_fold_cells(const float *values, const float *cell_value,
                                                                       const int *cell_index, int cells, int32_t *index) {
    __shared__ float pv[kArgmaxThreads / JL_WAVE];
    __shared__ int pi[kArgmaxThreads / JL_WAVE];
    const int tid = threadIdx.x;
    float best = -INFINITY;
    int at = INT_MAX;
    for (int i = tid; i < cells; i += kArgmaxThreads) keep_better(best, at, cell_value[i], cell_index[i]);
    fold_waves(best, at, pv, pi, tid, kArgmaxThreads / JL_WAVE);
    if (tid == 0) {
        if (at == INT_MAX || values[0] != values[0]) at = 0;   // as in jl_argmax_fold
        index[0] = at;
    }
}

// One lane per activation, 32 lanes per block: inverse = 127 / max|x| (0 for a block of zeros),
// q = (int)(x * inverse +- 0.5) clamped to +-127, scale = max|x| / 127, sum = sum of q.  With RMS
// the lane first computes its element of the normalised vector, rms_w[i] * (rms_scale * x[i]) with
// both products rounded to fp32, stores it to xb and quantises that
// (rmsApplyAndQuantizeActivationQ8Blocks, TransformerComputeKernelsQ4_0.java:374-432).
template <bool RMS>
__global__ void __launch_bounds__(256)
jl_quantize_q8_kernel(const float *__restrict__ x, const float *__restrict__ rms_w,
                      const float *__restrict__ rms_scale, float *__restrict__ xb, int64_t n,
                      int8_t *__restrict__ quants, float *__restrict__ scales, int32_t *__restrict__ sums) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    float value = i < n ? x[i] : 0.f;
    if constexpr (RMS) {
        if (i < n) {
            value = jl_mul_rn(rms_w[i], jl_mul_rn(rms_scale[0], value));
            xb[i] = value;
        }
    }
    float max_abs = fabsf(value);
#pragma unroll
    for (int o = 16; o > 0; o >>= 1) max_abs = fmaxf(max_abs, __shfl_xor(max_abs, o, JL_WAVE));
    const float inverse = max_abs > 0.0f ? __fdiv_rn(127.0f, max_abs) : 0.0f;
    const float scaled = jl_mul_rn(value, inverse);
    int q = (int)__fadd_rn(scaled, scaled >= 0.0f ? 0.5f : -0.5f);
    q = min(127, max(-127, q));
    int sum = q;
#pragma unroll
    for (int o = 16; o > 0; o >>= 1) sum += __shfl_xor(sum, o, JL_WAVE);
    if (i < n) {
        quants[i] = (int8_t)q;
        if ((i & 31) == 0) {
            scales[i >> 5] = __fdiv_rn(max_abs, 127.0f);
            sums[i >> 5] = sum;
        }
    }
}

// reductionOneBlock2WithLayer (J/backend/tornado/kernels/TransformerComputeKernelsLayered.java:570-580),
// the second phase of the unfused normalisation: output[i] = weights[i] * (ss * x[i]), both products
// rounded to fp32.
__global__ void __launch_bounds__(256)
jl_rms_apply_kernel(const float *__restrict__ x, const float *__restrict__ rms_w, const float *__restrict__ rms_scale,
                    float *__restrict__ xb, int64_t n) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) xb[i] = jl_mul_rn(rms_w[i], jl_mul_rn(rms_scale[0], x[i]));
}

}  // namespace

int jl_launch_rms_apply(jl_context *ctx, const float *x, const float *rms_w, const float *rms_scale, int64_t n,
                        float *xb) {
    hipLaunchKernelGGL(jl_rms_apply_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, ctx->stream, x, rms_w,
                       rms_scale, xb, n);
    JL_HIP(hipGetLastError());
    return JL_OK;
}

int jl_launch_rms_scale(jl_context *ctx, const float *x, int64_t n, float eps, float *scale) {
    hipLaunchKernelGGL(jl_rms_scale_kernel, dim3(1), dim3(kThreads), 0, ctx->stream, x, n, eps, scale);
    JL_HIP(hipGetLastError());
    return JL_OK;
}

static int argmax_launches(jl_context *ctx, const float *values, int64_t n, int32_t *index, ArgmaxCells *cells) {
    int groups = (int)((n / 4 + kArgmaxThreads - 1) / kArgmaxThreads);
    groups = groups < 1 ? 1 : groups > kArgmaxGroups ? kArgmaxGroups : groups;
    // the fold reads cells 0 .. groups - 1 only, all of them written by this call's scan: whatever an
    // earlier call left in the cells is never looked at, so nothing has to be cleared
    hipLaunchKernelGGL(jl_argmax_scan, dim3(groups), dim3(kArgmaxThreads), 0, ctx->stream, values, (int)n, cells);
    JL_HIP(hipGetLastError());
    hipLaunchKernelGGL(jl_argmax_fold, dim3(1), dim3(kArgmaxGroups), 0, ctx->stream, values, cells, groups, index);
    JL_HIP(hipGetLastError());
    return JL_OK;
}

int jl_launch_argmax(jl_context *ctx, const float *values, int64_t n, int32_t *index) {
    static_assert(sizeof(ArgmaxCells) <= JL_CONTEXT_SCRATCH_BYTES, "argmax cells exceed the context scratch");
    return argmax_launches(ctx, values, n, index, (ArgmaxCells *)ctx->scratch);
}

int jl_launch_argmax_rows(jl_context *ctx, const float *values, int64_t rows, int64_t n, int64_t row_stride,
                          int32_t *indices) {
    // a workgroup per row fills the chip from a few hundred rows on; smaller batches cut their rows
    // into runs (at most a wave's worth, and no more (run, row) cells than the context's scratch holds)
    int chunks = (int)(2 * ctx->compute_units / rows);
    if (chunks > JL_WAVE) chunks = JL_WAVE;
    if ((int64_t)chunks * rows > kProjectionCells) chunks = (int)(kProjectionCells / rows);
    if ((int64_t)chunks * 4096 > n) chunks = (int)(n / 4096);   // (runs of at least 4096 values)
    if (chunks < 2) {
        hipLaunchKernelGGL(jl_argmax_rows_kernel, dim3((unsigned)rows), dim3(kThreads), 0, ctx->stream, values, (int)n,
                           row_stride, indices);
        JL_HIP(hipGetLastError());
        return JL_OK;
    }
    float *cell_value = (float *)ctx->scratch;
    int *cell_index = (int *)(cell_value + kProjectionCells);
    hipLaunchKernelGGL(jl_argmax_rows_scan, dim3((unsigned)chunks, (unsigned)rows), dim3(kArgmaxThreads), 0, ctx->stream,
                       values, (int)n, row_stride, chunks, cell_value, cell_index);
    JL_HIP(hipGetLastError());
    hipLaunchKernelGGL(jl_argmax_rows_fold, dim3((unsigned)rows), dim3(JL_WAVE), 0, ctx->stream, values, row_stride, chunks,
                       cell_value, cell_index, indices);
    JL_HIP(hipGetLastError());
    return JL_OK;
}

int jl_launch_gemv_argmax(jl_context *ctx, const jl_weight *w, const float *x, const jl_rms *rms, float *out,
                          int32_t *index) {
    float *cell_value = (float *)ctx->scratch;
    jl_best_cells cells{cell_value, (int *)(cell_value + kProjectionCells), kProjectionCells};
    int st = jl_launch_gemv(ctx, &w, 1, &out, nullptr, x, JL_STORE, rms, nullptr, &cells);
    if (st == JL_NO_CELLS_FORM) {
        // a shape or type whose kernel keeps no cells: the projection, then the scan over its output
        st = jl_launch_gemv(ctx, &w, 1, &out, nullptr, x, JL_STORE, rms);
        if (st != JL_OK) return st;
        return jl_launch_argmax(ctx, out, w->rows, index);
    }
    if (st != JL_OK) return st;
    hipLaunchKernelGGL(jl_argmax_fold_cells, dim3(1), dim3(kArgmaxThreads), 0, ctx->stream, out, cells.value, cells.index,
                       cells.count, index);
    JL_HIP(hipGetLastError());
    return JL_OK;
}

// ---- jl_argmax_static: the same two launches with the cells in a device array of the library ----
//
// `scratch` lives in the code object: every device the library runs on holds its own copy at its
// own address from the moment the code object is loaded there until the process ends.  In host code
// the name is only a handle for hipGetSymbolAddress; the kernels take the address that call returns.
#define JL_STATIC_SCRATCH_BYTES 1024
static __device__ __align__(256) unsigned char scratch[JL_STATIC_SCRATCH_BYTES];
static_assert(sizeof(ArgmaxCells) <= JL_STATIC_SCRATCH_BYTES, "argmax cells exceed the static scratch");

static void *g_static_scratch[JL_MAX_DEVICES] = {};   // device address of `scratch`, per device

int jl_static_scratch_init(int device) {
    if (device < 0 || device >= JL_MAX_DEVICES) return JL_OK;   // such a device simply has no jl_argmax_static
    if (__atomic_load_n(&g_static_scratch[device], __ATOMIC_ACQUIRE)) return JL_OK;
    void *ptr = nullptr;
    JL_HIP(hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)));   // the caller made `device` current
    if (!ptr) return jl_fail(JL_ERR_HIP, "hipGetSymbolAddress returned a null address for the static scratch");
    __atomic_store_n(&g_static_scratch[device], ptr, __ATOMIC_RELEASE);
    return JL_OK;
}

int jl_launch_argmax_static(jl_context *ctx, const float *values, int64_t n, int32_t *index) {
    void *cells = ctx->device >= 0 && ctx->device < JL_MAX_DEVICES
                      ? __atomic_load_n(&g_static_scratch[ctx->device], __ATOMIC_ACQUIRE) : nullptr;
    if (!cells) {
        return jl_fail(JL_ERR_UNSUPPORTED, "jl_argmax_static: device %d has no static scratch (the library keeps one "
                       "for devices 0..%d, set up by jl_context_create)", ctx->device, JL_MAX_DEVICES - 1);
    }
    return argmax_launches(ctx, values, n, index, (ArgmaxCells *)cells);
}

namespace {

// One workgroup of 256 per activation row, and the reference kernel's own summation order (its
// local size is 256 too): thread t adds the squares of elements t, t + 256, ... in turn -- product
// rounded, then the sum -- and the 256 partial sums fold as the tree partial[t] += partial[t + s],
// s = 128 ... 1.  With correctly rounded division and square root the scale, and so every fp16
// output, has the bits the reference's source states.  Rows of up to 8192 columns are read once.
// ADD: the pending residual add first, batchedRmsReduceFusedResidual (:1519-1551): x += delta is
// written back and everything after it runs over the updated row.
template <int STEPS, bool ADD>
__global__ void __launch_bounds__(256)
jl_rms_apply_f16_kernel(float *__restrict__ X, const float *__restrict__ delta, const float *__restrict__ w,
                        float eps, int n, float *__restrict__ scales, _Float16 *__restrict__ out) {
    __shared__ float partial[256];
    const int tid = threadIdx.x;
    float *x = X + (int64_t)blockIdx.x * n;
    const float *dl = ADD ? delta + (int64_t)blockIdx.x * n : nullptr;
    _Float16 *o = out + (int64_t)blockIdx.x * n;
    // STEPS > 0: the row fits STEPS elements per thread and is read once; every load goes out
    // before the first sum needs one (a load and its use inside one predicated step would make
    // the steps wait for each other: a round trip to memory per step)
    constexpr int HELD = STEPS > 0 ? STEPS : 1;
    float v[HELD], wv[HELD];
    float ss = 0.f;
    if constexpr (STEPS > 0) {
#pragma unroll
        for (int j = 0; j < HELD; j++) {
            const int i = tid + j * 256;
            v[j] = x[i < n ? i : 0];
        }
#pragma unroll
        for (int j = 0; j < HELD; j++) {
            const int i = tid + j * 256;
            wv[j] = w[i < n ? i : 0];
        }
        if constexpr (ADD) {
            float dv[HELD];
#pragma unroll
            for (int j = 0; j < HELD; j++) {
                const int i = tid + j * 256;
                dv[j] = dl[i < n ? i : 0];
            }
#pragma unroll
            for (int j = 0; j < HELD; j++) {
                const int i = tid + j * 256;
                v[j] = __fadd_rn(v[j], dv[j]);
                if (i < n) x[i] = v[j];
            }
        }
#pragma unroll
        for (int j = 0; j < HELD; j++) {
            const float next = __fadd_rn(ss, jl_mul_rn(v[j], v[j]));
            ss = tid + j * 256 < n ? next : ss;
        }
    } else {
        for (int i = tid; i < n; i += 256) {
            float xi = x[i];
            if constexpr (ADD) {
                xi = __fadd_rn(xi, dl[i]);
                x[i] = xi;
            }
            ss = __fadd_rn(ss, jl_mul_rn(xi, xi));
        }
    }
    partial[tid] = ss;
    __syncthreads();
    for (int s = 128; s > 0; s >>= 1) {
        if (tid < s) partial[tid] = __fadd_rn(partial[tid], partial[tid + s]);
        __syncthreads();
    }
    const float m = __fadd_rn(__fdiv_rn(partial[0], (float)n), eps);
    // (the square root through double: correctly rounded to fp32, which __fsqrt_rn is not here)
    const float scale = __fdiv_rn(1.0f, (float)sqrt((double)m));
    if (tid == 0 && scales) scales[blockIdx.x] = scale;
    if constexpr (STEPS > 0) {
#pragma unroll
        for (int j = 0; j < HELD; j++) {
            const int i = tid + j * 256;
            if (i < n) o[i] = (_Float16)jl_mul_rn(jl_mul_rn(wv[j], scale), v[j]);
        }
    } else {
        for (int i = tid; i < n; i += 256) o[i] = (_Float16)jl_mul_rn(jl_mul_rn(w[i], scale), x[i]);
    }
}

}  // namespace

template <bool ADD>
static void launch_rms_apply(jl_context *ctx, float *X, const float *delta, const float *w, float eps, int64_t rows,
                             int n, float *scales, _Float16 *out) {
    const dim3 g((unsigned)rows), b(256);
    if (n <= 8 * 256) hipLaunchKernelGGL((jl_rms_apply_f16_kernel<8, ADD>), g, b, 0, ctx->stream, X, delta, w, eps, n, scales, out);
    else if (n <= 16 * 256) hipLaunchKernelGGL((jl_rms_apply_f16_kernel<16, ADD>), g, b, 0, ctx->stream, X, delta, w, eps, n, scales, out);
    else if (n <= 32 * 256) hipLaunchKernelGGL((jl_rms_apply_f16_kernel<32, ADD>), g, b, 0, ctx->stream, X, delta, w, eps, n, scales, out);
    else hipLaunchKernelGGL((jl_rms_apply_f16_kernel<0, ADD>), g, b, 0, ctx->stream, X, delta, w, eps, n, scales, out);
}

int jl_launch_rms_apply_f16(jl_context *ctx, float *X, const float *delta, const float *w, float eps, int64_t rows,
                            int64_t n, float *scales, _Float16 *out) {
    if (delta) launch_rms_apply<true>(ctx, X, delta, w, eps, rows, (int)n, scales, out);
    else launch_rms_apply<false>(ctx, X, delta, w, eps, rows, (int)n, scales, out);
    JL_HIP(hipGetLastError());
    return JL_OK;
}

int jl_launch_quantize_q8(jl_context *ctx, const float *x, const float *rms_w, const float *rms_scale, float *xb,
                          int64_t n, int8_t *quants, float *scales, int32_t *sums) {
    const dim3 g((unsigned)((n + 255) / 256)), b(256);
    if (rms_w) {
        hipLaunchKernelGGL(jl_quantize_q8_kernel<true>, g, b, 0, ctx->stream, x, rms_w, rms_scale, xb, n, quants,
                           scales, sums);
    } else {
        hipLaunchKernelGGL(jl_quantize_q8_kernel<false>, g, b, 0, ctx->stream, x, rms_w, rms_scale, xb, n, quants,
                           scales, sums);
    }
    JL_HIP(hipGetLastError());
    return JL_OK;
}
