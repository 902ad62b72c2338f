// Host-side internals shared by the translation units of libjitllm_hip.so.
#pragma once

#include <hip/hip_runtime.h>
#include <atomic>
#include <stdint.h>
#include <stdio.h>

#include "../../include/jitllm_hip.h"

struct jl_context {
    int device;
    hipStream_t stream;
    bool owns_stream;
    int compute_units;
    char name[128];
    void *scratch;   // JL_CONTEXT_SCRATCH_BYTES of device memory for results handed from one launch of
                     // a call to the next (calls on a context are ordered on its stream)
    // JL_CONTEXT_ARRIVALS counters, all zero between calls: the workgroups of a batched-decode launch
    // that share a set of output rows count themselves in here, and the last one to arrive folds
    // their partial sums (and puts the counter back to zero).
    uint32_t *arrivals;
    // Pinned host memory that jl_upload / jl_download stage the caller's pageable memory through, two
    // halves in turn: every transfer the device sees is then a DMA from / to pinned memory, and the
    // caller's pointer is only ever touched by a host memcpy.
    uint8_t *bounce;
    hipEvent_t bounce_done[2];
    // false: no GEMM of this context cuts K across work items (jl_context_set_split_k), so that a
    // row's sums are added in one order whatever the call's row count
    bool split_k = true;
};
#define JL_CONTEXT_SCRATCH_BYTES 8192
#define JL_CONTEXT_ARRIVALS 1024
#define JL_BOUNCE_HALF_BYTES (8u << 20)

struct jl_weight {
    jl_context *ctx;
    int type;
    int64_t rows;
    int64_t cols;
    int64_t bytes;
    const uint8_t *blocks;  // device address of the first block
    bool owns_blocks;
};

// Block geometry (reference: J/format/GGMLType.java:7,13,18-20).
static inline int jl_block_elems(int type) {
    switch (type) {
        case JL_Q4_K: case JL_Q5_K: case JL_Q6_K: case JL_IQ4_XS: return 256;
        case JL_Q8_0: case JL_Q4_0: case JL_Q4_1: case JL_Q5_0: return 32;
        default: return 0;
    }
}
static inline int jl_block_bytes(int type) {
    switch (type) {
        case JL_Q4_0: return 18;
        case JL_Q4_1: return 20;
        case JL_Q5_0: return 22;
        case JL_Q8_0: return 34;
        case JL_Q4_K: return 144;
        case JL_Q5_K: return 176;
        case JL_Q6_K: return 210;
        case JL_IQ4_XS: return 136;
        default: return 0;
    }
}
static inline const char *jl_type_name(int type) {
    switch (type) {
        case JL_Q4_0: return "Q4_0";
        case JL_Q4_1: return "Q4_1";
        case JL_Q5_0: return "Q5_0";
        case JL_Q8_0: return "Q8_0";
        case JL_Q4_K: return "Q4_K";
        case JL_Q5_K: return "Q5_K";
        case JL_Q6_K: return "Q6_K";
        case JL_IQ4_XS: return "IQ4_XS";
        default: return "?";
    }
}
// Q8_0, Q4_0 and Q4_K have the whole kernel family; Q4_1, Q5_0, Q5_K, Q6_K and IQ4_XS the plain
// single-token projection and the decode-once batched path.
static inline bool jl_has_fused_kernels(int type) {
    return type == JL_Q8_0 || type == JL_Q4_0 || type == JL_Q4_K;
}

// Records the calling thread's error message and returns `status`.
int jl_fail(int status, const char *fmt, ...) __attribute__((format(printf, 2, 3)));

#define JL_HIP(call)                                                                      \
    do {                                                                                  \
        hipError_t e_ = (call);                                                           \
        if (e_ != hipSuccess)                                                             \
            return jl_fail(e_ == hipErrorOutOfMemory ? JL_ERR_OOM : JL_ERR_HIP,           \
                           "%s failed: %s", #call, hipGetErrorString(e_));                \
    } while (0)

// Raises a kernel's limit of dynamic LDS, once per kernel and device: `done` is the launcher's own
// static array of flags, one per device index (contexts on several host threads may come through
// here at once; an index past the array is configured on every call).
struct jl_lds_limit_flags {
    std::atomic<bool> done[16];
};
inline int jl_raise_lds_limit(jl_lds_limit_flags &flags, int device, const void *kernel, int bytes) {
    const bool tracked = device >= 0 && device < 16;
    if (tracked && flags.done[device].load(std::memory_order_acquire)) return JL_OK;
    JL_HIP(hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, bytes));
    if (tracked) flags.done[device].store(true, std::memory_order_release);
    return JL_OK;
}

#define JL_REQUIRE(cond, ...)                                  \
    do {                                                       \
        if (!(cond)) return jl_fail(JL_ERR_INVALID, __VA_ARGS__); \
    } while (0)

// Launchers implemented per translation unit; each returns a jl_status.
int jl_launch_dequant(jl_context *ctx, const jl_weight *w, float *out);
// RMS normalisation folded into a projection's activation load: x_j -> weights[j] * (s * x_j), with
// s = scale[0] (device) or, when scale is null, 1 / sqrt(sum x^2 / n + eps) computed by the kernel.
struct jl_rms {
    const float *weights;
    const float *scale;
    float eps;
};
// The activation as Q8 blocks (jl_quantize_q8): 32 signed bytes, a scale and the bytes' sum per block.
struct jl_q8x {
    const int8_t *quants;
    const float *scales;
    const int32_t *sums;
};
// Per-workgroup (largest stored output, its row) cells of a projection, for greedy sampling:
// `count` is the room going in and the cells written coming out.
struct jl_best_cells {
    float *value;
    int *index;
    int count;
};
#define JL_NO_CELLS_FORM 1   // jl_launch_gemv with `cells`: this launch has no such form, nothing was launched
// `xq` set: the packed-integer kernels read it instead of `x`.  `cells` set (one weight, JL_STORE):
// the kernel also leaves them, or the call returns JL_NO_CELLS_FORM.
int jl_launch_gemv(jl_context *ctx, const jl_weight *const *w, int nseg, float *const *outs,
                   const jl_weight *w_up, const float *x, int epilogue, const jl_rms *rms,
                   const jl_q8x *xq = nullptr, jl_best_cells *cells = nullptr);
// `rms_w` set: xb = rms_w * (rms_scale[0] * x) is written and quantised instead of x.
int jl_launch_quantize_q8(jl_context *ctx, const float *x, const float *rms_w, const float *rms_scale, float *xb,
                          int64_t n, int8_t *quants, float *scales, int32_t *sums);
int jl_launch_rms_apply_f16(jl_context *ctx, float *X, const float *delta, const float *w, float eps, int64_t rows,
                            int64_t n, float *scales, _Float16 *out);
// `w_up` set: out = SiLU(w . x) * (w_up . x) (the fused gate/up), `epilogue` ignored.
int jl_launch_gemv_direct(jl_context *ctx, const jl_weight *w, const jl_weight *w_up, const float *x, float *out,
                          int epilogue);
int jl_launch_dequant_direct(jl_context *ctx, const jl_weight *w, float *out);
int jl_launch_rms_scale(jl_context *ctx, const float *x, int64_t n, float eps, float *scale);
int jl_launch_rms_apply(jl_context *ctx, const float *x, const float *rms_w, const float *rms_scale, int64_t n,
                        float *xb);
int jl_launch_argmax(jl_context *ctx, const float *values, int64_t n, int32_t *index);
int jl_launch_argmax_rows(jl_context *ctx, const float *values, int64_t rows, int64_t n, int64_t row_stride,
                          int32_t *indices);
// out = w . x (rms set: the normalisation folded in) and index[0] = the first maximum of out.
int jl_launch_gemv_argmax(jl_context *ctx, const jl_weight *w, const float *x, const jl_rms *rms, float *out,
                          int32_t *index);
// jl_argmax with its (value, index) cells in a device array that is part of the library's code
// object instead of the context's allocation.  jl_static_scratch_init looks that array's address
// up on the current device (once per device; jl_context_create calls it).
#define JL_MAX_DEVICES 64
int jl_static_scratch_init(int device);
int jl_launch_argmax_static(jl_context *ctx, const float *values, int64_t n, int32_t *index);
int jl_launch_swiglu(jl_context *ctx, float *gate, const float *up, int64_t count);
int jl_launch_residual_add(jl_context *ctx, float *residual, const float *delta, int64_t count);
int jl_launch_fill(jl_context *ctx, float *dst, float value, size_t count);
// A caller-owned fp16 copy of one projection's weights that outlives the call: decoded when
// *state does not name the layout the call needs (0 = empty), reused otherwise.
struct jl_resident {
    void *copy;
    size_t bytes;
    int32_t *state;
};
// Activations that arrive as binary16 (`x16`, read instead of X) and a SWIGLU result wanted as
// binary16 (`c_f16`: C is then an array of binary16 values).
struct jl_half_io {
    const _Float16 *x16;
    bool c_f16;
};
int jl_launch_gemm(jl_context *ctx, const jl_weight *const *weights, int count, const float *X,
                   float *C, int64_t batch, int64_t active_rows, int64_t ldo, int64_t col_offset,
                   int epilogue, int math, void *workspace, size_t workspace_bytes,
                   const jl_resident *resident, const jl_half_io *half = nullptr);
// Batched decode (at most 64 rows; up to 511 where priced cheaper, see `other_us`): the weight-streaming kernel.  `taken` says whether the shape
// was one it handles; when not, nothing was launched and the tiled GEMM must run instead.  `X16`
// set: the activations as binary16 (X is then ignored); `c_f16` (JL_SWIGLU): C holds binary16.
// `other_us`: what the caller's other way of running a call of 65 .. 511 rows is estimated to take,
// in microseconds; such a call is taken only when streaming is estimated cheaper.
int jl_launch_gemm_skinny(jl_context *ctx, const jl_weight *const *weights, int count, const float *X,
                          const _Float16 *X16, float *C, bool c_f16, int rows, int64_t ldo, int64_t col_offset,
                          int epilogue, float *planes, size_t plane_bytes, double other_us, bool *taken);
// Activation rows one of its workgroups multiplies: 16 or 32; calls of more rows run as two row blocks.
int jl_skinny_padded_rows(int rows);
// (its two halves, one translation unit each: fp32 activations, binary16 activations)
int jl_launch_gemm_skinny_x32(jl_context *ctx, const jl_weight *const *weights, int count, const float *X,
                              const _Float16 *X16, float *C, bool c_f16, int rows, int64_t ldo, int64_t col_offset,
                              int epilogue, float *planes, size_t plane_bytes, double other_us, bool *taken);
int jl_launch_gemm_skinny_x16(jl_context *ctx, const jl_weight *const *weights, int count, const float *X,
                              const _Float16 *X16, float *C, bool c_f16, int rows, int64_t ldo, int64_t col_offset,
                              int epilogue, float *planes, size_t plane_bytes, double other_us, bool *taken);
// Many-row prefill: weights decoded to fp16 once per call into `copy`, then a plain fp16 GEMM.
int jl_dense_column_tile(int rows, int k, int out_cols_virtual, int epilogue, int compute_units, int *splits,
                         int *row_tile, int min_rows = 512, bool may_cut_k = true);
size_t jl_dense_copy_bytes(int k, int out_cols_virtual);
size_t jl_dense_plane_bytes(int rows, int out_cols_virtual, int splits);
int jl_launch_gemm_dense(jl_context *ctx, const jl_weight *const *weights, int count, const _Float16 *A,
                         const float *row_scale, float *C, int rows, int64_t ldo, int64_t col_offset,
                         int epilogue, _Float16 *copy, bool decode, int bm, int bn, int splits, float *planes,
                         bool c_f16 = false, const float *X32 = nullptr, float *row_scale_out = nullptr);
// Adds split-K planes [splits][rows padded][ntiles * 128] in split order and applies the epilogue.
int jl_launch_gemm_reduce(jl_context *ctx, const float *planes, const float *row_scale, float *C, int rows,
                          int n_total, int ntiles, int64_t plane, int splits, int64_t ldo, int64_t col_offset,
                          int epilogue);
// JL_MATH_INT8: activations quantised per 32-block, int8 MFMA over the raw Q8_0 / Q4_0 blocks, one
// fp32 scale product per block in k order.
size_t jl_gemm_i8_workspace_bytes(int64_t max_rows, int64_t cols);
int jl_launch_gemm_i8(jl_context *ctx, const jl_weight *const *weights, int count, const float *X, float *C,
                      int64_t batch, int rows, int64_t ldo, int64_t col_offset, int epilogue, void *workspace,
                      size_t workspace_bytes);
size_t jl_gemm_workspace_bytes_impl(int64_t max_rows, int64_t cols, int64_t out_cols, int math);
