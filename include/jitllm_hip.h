/*
 * jitllm_hip.h -- C ABI of libjitllm_hip.so: jitLLM's quantized weight projections on one MI355X.
 *
 * The library replaces, inside a forward pass, the TornadoVM tasks behind three Java seams of the
 * reference (J = src/main/java/org/beehive/jitllm):
 *   decode          J/backend/tornado/layers/QuantizedProjections.java        (matvec, floatMatvec,
 *                   residualMatvec, gateUp, and the fused q|k|v kernels its layer builders call)
 *   batched decode  J/backend/tornado/layers/QuantizedBatchProjections.java   (projection, gateUp)
 *   batched prefill J/backend/tornado/ops/Implementation.java + Instance.java (needs/create/emit)
 * Weights are GGUF blocks in the file's own layout (Q8_0 34 B / 32, Q4_0 18 B / 32, Q4_K 144 B /
 * 256; J/format/GGMLType.java:7,13,18-20), uploaded once and never converted.  Activations and
 * outputs are fp32 device buffers that the caller owns and rebinds by value, never by address
 * (the batched prefill also takes and leaves the fp16 buffers of the reference's plan: jl_gemm_xf16).
 *
 * Conventions
 *   - every entry point returns JL_OK (0) or a negative jl_status; jl_last_error() then names the
 *     cause on the calling thread.  Nothing falls back silently: an unsupported combination is
 *     JL_ERR_UNSUPPORTED, never a slower path computing something else.
 *   - `n` is the row length (input features), `d` the row count (output features), as in the
 *     reference's kernels.  A `[d x n]` weight is d rows of n / block_elems blocks, row-major.
 *   - all work is enqueued on the context's HIP stream and is ordered on it; no entry point below
 *     jl_weight_upload / jl_malloc allocates device memory.
 *   - a context is used by one host thread at a time (the reference's sessions are
 *     single-threaded: docs/architecture/memory-and-concurrency.md:101-115).
 */
#ifndef JITLLM_HIP_H
#define JITLLM_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define JL_ABI_VERSION 1

typedef enum jl_status {
    JL_OK = 0,
    JL_ERR_INVALID = -1,     /* bad argument: null pointer, shape that is not whole blocks, ... */
    JL_ERR_UNSUPPORTED = -2, /* combination with no kernel (IllegalStateException "no ... kernel for") */
    JL_ERR_HIP = -3,         /* a HIP runtime call failed; the message carries hipGetErrorString */
    JL_ERR_OOM = -4,         /* device allocation failed (the reference's GPUL-MEM-001) */
    JL_ERR_WORKSPACE = -5    /* caller's workspace smaller than jl_gemm_workspace_bytes asked for */
} jl_status;

/* ggml type ids as a GGUF tensor-info record carries them (GGMLType ordinals). */
/* Q8_0, Q4_0 and Q4_K have every entry point below.  Q6_K (210 B / 256) and Q5_K (176 B / 256;
 * J/format/GGMLType.java:21-29: the vocabulary projection and some attention / feed-forward tensors
 * of "Q4_K_M" files are Q6_K, "Q5_K_M" files are Q5_K with Q6_K), and the types quantisers mix
 * into other files -- Q4_1 (20 B / 32, GGMLType.java:8), Q5_0 (22 B / 32, :11) and IQ4_XS
 * (136 B / 256, :39-41) -- have
 * jl_dequant_f32, jl_gemv, jl_gemv_gate_up and jl_gemm -- the latter on the weight-streaming kernel
 * at up to 64 rows -- and up to 511 where that is the faster way -- and by decoding the weights to fp16 into the workspace
 * first above that.  (Of these the reference fuses gate/up
 * for Q5_K only, QuantizedProjections.java:386-393; the one-launch form is there for all five.)  The
 * fused q|k|v, RMS-folding and packed-activation single-token entry points return
 * JL_ERR_UNSUPPORTED for them; a caller that gets JL_ERR_UNSUPPORTED runs the unfused steps. */
typedef enum jl_ggml_type {
    JL_Q4_0 = 2, JL_Q4_1 = 3, JL_Q5_0 = 6, JL_Q8_0 = 8, JL_Q4_K = 12, JL_Q5_K = 13, JL_Q6_K = 14, JL_IQ4_XS = 23
} jl_ggml_type;

/* What a projection does with its result (Int8GemmKernels.java:617-621 EPILOGUE_*). */
typedef enum jl_epilogue {
    JL_STORE = 0,    /* out  = W.x                                                   */
    JL_RESIDUAL = 1, /* out += W.x   (matrixVectorGenericWithResidual*, residualMatvec) */
    JL_SWIGLU = 2    /* out  = SiLU(W1.x) * (W3.x), SiLU(g) = g / (1 + exp(-g))       */
} jl_epilogue;

/* Arithmetic of the batched GEMM (jl_gemm). */
typedef enum jl_gemm_math {
    JL_MATH_DEFAULT = 0, /* JL_MATH_F16 for every type                                         */
    JL_MATH_F16 = 1,     /* weights decoded to fp16 in LDS, activations rounded to fp16, fp32  */
                         /* accumulation on fp16 MFMA (TransformerBatchPrefillKernels gemmMMAQ8) */
    JL_MATH_INT8 = 2     /* activations quantised per 32-block to int8, int8 MFMA, one fp32     */
                         /* scale product per block (Int8GemmKernels.java:17-23); Q8_0 and Q4_0 */
} jl_gemm_math;

typedef struct jl_context jl_context;
typedef struct jl_weight jl_weight;

int jl_abi_version(void);
const char *jl_last_error(void);

/* ---- context: one device, one stream ------------------------------------------------------- */

/* Creates a context on `device` with a stream of its own (default priority). */
int jl_context_create(int device, jl_context **out);
/* Same, on a stream the caller owns (a hipStream_t); the stream is borrowed, never destroyed. */
int jl_context_create_on_stream(int device, void *hip_stream, jl_context **out);
int jl_context_destroy(jl_context *ctx);
/* Blocks until everything enqueued on the context's stream has finished. */
int jl_sync(jl_context *ctx);
void *jl_context_stream(jl_context *ctx);
/* Compute units of the device and its name (DeviceCapability of the reference's backend SPI). */
int jl_device_info(jl_context *ctx, int *compute_units, char *name, size_t name_bytes);
/*
 * enabled == 0: no jl_gemm* call on this context cuts K across work items; every GEMM stays whole,
 * as under the reference's -Djitllm.prefill.splitK=false (SplitKGemm.java:40-42,
 * J/backend/tornado/layers/).  A narrow output at few rows (a 2048-wide projection of a 512-token
 * chunk) is otherwise computed as 2, 4 or 8 runs of K whose partial sums are added afterwards: faster,
 * and a different order of addition than the same rows get in a larger chunk.  With the switch off
 * a prefill row's result does not depend on how many rows (>= 512) share its call.  Default: on.
 * Batched decode (calls of up to 64 rows) is not affected.
 */
int jl_context_set_split_k(jl_context *ctx, int enabled);

/* ---- device buffers for fp32 activations (TornadoVM FloatArray of the reference) ----------- */

int jl_malloc(jl_context *ctx, size_t bytes, void **device_ptr);
int jl_free(jl_context *ctx, void *device_ptr);
/* Stream-ordered copies; the host side has returned only after the copy completed.  The host
 * pointer may be pageable (a heap segment, a mapped file): it is copied through pinned staging
 * memory the context owns, 8 MiB at a time, so neither call is legal inside a stream capture. */
int jl_upload(jl_context *ctx, void *device_dst, const void *host_src, size_t bytes);
int jl_download(jl_context *ctx, void *host_dst, const void *device_src, size_t bytes);
/* Fills `count` floats with `value` (FloatArray.init). */
int jl_fill_f32(jl_context *ctx, float *device_dst, float value, size_t count);

/* ---- weights (TornadoTensor: J/backend/tornado/tensor/TornadoTensor.java:17-101) ----------- */

/*
 * Uploads the raw blocks of a `[rows x cols]` weight as the GGUF file stores them, with no
 * conversion (ModelLoader.loadTornadoTensorNative, J/model/loader/ModelLoader.java:246-290).
 * `host_blocks` points at the first block, i.e. past the 16-byte array header the reference's
 * mmapped segments carry (TornadoTensorLoader.java:42-44).
 */
int jl_weight_upload(jl_context *ctx, int ggml_type, const void *host_blocks, int64_t rows,
                     int64_t cols, jl_weight **out);
/* Wraps blocks already resident in device memory (16-byte aligned); nothing is copied or owned. */
int jl_weight_wrap(jl_context *ctx, int ggml_type, const void *device_blocks, int64_t rows,
                   int64_t cols, jl_weight **out);
int jl_weight_free(jl_weight *w);
int jl_weight_info(const jl_weight *w, int *ggml_type, int64_t *rows, int64_t *cols,
                   int64_t *bytes);
/* Device address of the blocks (TornadoTensor.asByteArray). */
const void *jl_weight_blocks(const jl_weight *w);

/*
 * Decodes every element to fp32 with the host tensor's own arithmetic -- bit for bit what
 * Q8_0FloatTensor.getFloat (Q8_0FloatTensor.java:52-61), Q4_0FloatTensor.getFloat
 * (Q4_0FloatTensor.java:55-79) and Q4_KFloatTensor.getFloat (Q4_KFloatTensor.java:87-122) return.
 * `out` holds rows * cols floats.  The parity probe; also dequantize*ToFP16's fp32 sibling.
 */
int jl_dequant_f32(jl_context *ctx, const jl_weight *w, float *out);

/* ---- decode: one activation vector (QuantizedProjections.java) ----------------------------- */

/*
 * out = W.x (JL_STORE; QuantizedProjections.floatMatvec :200-254, matrixVectorGenericQ8Byte,
 * matrixVectorGenericQ4_0, matrixVectorGenericQ4_K) or out += W.x (JL_RESIDUAL;
 * QuantizedProjections.residualMatvec :260-379).  x holds cols floats, out rows floats.
 */
int jl_gemv(jl_context *ctx, const jl_weight *w, const float *x, float *out, int epilogue);

/*
 * q = Wq.x, k = Wk.x, v = Wv.x in one launch (fusedQKVMatmulQ8,
 * TransformerComputeKernelsLayered.java:2488+; fusedQKVMatmulQ4_0; fusedQKVMatmulQ4_KNonSquare).
 * The three weights share the type and the row length.
 */
int jl_gemv_qkv(jl_context *ctx, const jl_weight *wq, const jl_weight *wk, const jl_weight *wv,
                const float *x, float *q, float *k, float *v);

/*
 * hb = SiLU(W1.x) * (W3.x) in one launch (fusedFeedForwardWithSiLUAndGLUActivationQ8_0Byte,
 * TransformerComputeKernelsLayered.java:2453-2479; fusedFFNGateUpSiLUQ4_0; fusedFFNGateUpSiLUQ4_K;
 * the Q5_K sibling; QuantizedProjections.gateUp :400-480).  Every weight type with a jl_gemv has
 * it.  Both weights share type and shape; a mixed pair is JL_ERR_UNSUPPORTED and the caller runs
 * two jl_gemv and jl_swiglu, as the reference does.
 */
int jl_gemv_gate_up(jl_context *ctx, const jl_weight *w1, const jl_weight *w3, const float *x,
                    float *hb);

/* gate[i] = SiLU(gate[i]) * up[i] (siluAndMultiply; the unfused tail of gateUp). */
int jl_swiglu(jl_context *ctx, float *gate, const float *up, int64_t count);
/*
 * residual[i] += delta[i]: batchedResidualAddFP32 (TransformerBatchPrefillKernels.java:1078-1084), the
 * prefill plan's "residual add" step where a family runs a task of its own between the down
 * projection and the add (TensorCoreSteps.java:70-75); a down projection that is followed by its add
 * directly is one jl_gemm call with JL_RESIDUAL instead.
 */
int jl_residual_add(jl_context *ctx, float *residual, const float *delta, int64_t count);

/* ---- the steps on either side of a decode projection ------------------------------------------ */

/*
 * scale[0] = (float)(1 / sqrt(sum_j x[j]^2 / n + eps)), a device scalar: the factor
 * CpuOperations.rmsnorm applies (J/inference/op/CpuOperations.java:60-66) and what
 * reductionOneBlockWithLayer leaves for the fused kernels
 * (J/backend/tornado/kernels/TransformerComputeKernels.java:378-437).  The sum is taken in parallel,
 * so its last bits may differ from the host's sequential sum.
 */
int jl_rms_scale(jl_context *ctx, const float *x, int64_t n, float eps, float *scale);
/*
 * xb[i] = rms_weights[i] * (rms_scale[0] * x[i]), both products rounded to fp32: the second phase of
 * the unfused normalisation, reductionOneBlock2WithLayer
 * (J/backend/tornado/kernels/TransformerComputeKernelsLayered.java:570-580), which
 * QuantizedProjections.rmsApply dispatches where the projections are not packed
 * (QuantizedProjections.java:117-130).  For the steps that have no RMS-folding launch -- projections
 * over Q6_K, Q5_K, Q4_1, Q5_0 and IQ4_XS weights, row lengths the folding kernels refuse.  xb may be x.
 */
int jl_rms_apply(jl_context *ctx, const float *x, const float *rms_weights, const float *rms_scale, int64_t n,
                 float *xb);

/*
 * The projections above with the RMS normalisation of x folded into the activation load:
 * x_j is replaced by rms_weights[j] * (s * x_j) (CpuOperations.rmsnorm :67-72) and never written
 * back.  s = rms_scale[0], a device scalar such as jl_rms_scale leaves (fusedRmsNormQKVMatmulQ8,
 * TransformerComputeKernelsLayered.java:2116-2220; reductionOneBlock2WithLogits + the vocabulary
 * projection, TransformerComputeKernels.java:439-444, LogitsQ8_0Layer.java:85-97); or, with
 * rms_scale null, s = 1 / sqrt(sum x^2 / n + eps) computed from x by every workgroup for itself,
 * which saves the reduction's launch (fullyFusedRmsNormFFNGateUpQ8,
 * TransformerComputeKernelsLayered.java:2866+, always works this way: jl_gemv_gate_up_rms).
 * Row length: a multiple of 64 up to 16384 (8192 for gate/up, whose tile holds a row of each
 * matrix), x and rms_weights 16-byte aligned; otherwise
 * JL_ERR_UNSUPPORTED and the caller normalises first, as the unfused reference path does.
 */
int jl_gemv_rms(jl_context *ctx, const jl_weight *w, const float *x, const float *rms_weights,
                const float *rms_scale, float eps, float *out, int epilogue);
int jl_gemv_qkv_rms(jl_context *ctx, const jl_weight *wq, const jl_weight *wk, const jl_weight *wv,
                    const float *x, const float *rms_weights, const float *rms_scale, float eps,
                    float *q, float *k, float *v);
int jl_gemv_gate_up_rms(jl_context *ctx, const jl_weight *w1, const jl_weight *w3, const float *x,
                        const float *rms_weights, float eps, float *hb);

/*
 * index[0] = position of the first maximum of values[0..n) (device int32): greedy sampling without
 * bringing the logits to the host (argmaxLogits, TransformerComputeKernels.java:95-127;
 * FloatTensor.argmax, J/tensor/standard/FloatTensor.java:168-181, whose tie and NaN behaviour --
 * first of equals, 0 when element 0 is NaN -- this follows).
 */
int jl_argmax(jl_context *ctx, const float *values, int64_t n, int32_t *index);
/*
 * The same for the logits of a batch: indices[b] = position of the first maximum of
 * values[b * row_stride .. + n), b < rows, in one launch -- batchedArgmaxLogits
 * (J/backend/tornado/kernels/TransformerBatchPrefillKernels.java:2118-2159), the last task of the
 * batched logits graph (J/backend/tornado/batch/TornadoBatchExecutor.java:226-232), so that only
 * `rows` integers cross to the host.  Ties and NaN as jl_argmax (the reference kernel's tree keeps
 * whichever of two equal maxima its lower thread held; the host's scan, followed here, the first).
 */
int jl_argmax_rows(jl_context *ctx, const float *values, int64_t rows, int64_t n, int64_t row_stride,
                   int32_t *indices);

/*
 * The tail of a greedy decode step in one call: out = w . x, the vocabulary projection -- with the
 * final RMS normalisation folded in as in jl_gemv_rms when rms_weights is set (rms_scale and eps as
 * there), x used as it is when rms_weights is null -- and index[0] = jl_argmax(out) (the
 * vocabulary projection followed by "argmax_sample", LogitsQ8_0Layer.java:92-110,
 * LogitsFP16Layer.java:217).  out and index[0] are bit for bit what jl_gemv / jl_gemv_rms followed
 * by jl_argmax leave.  A Q8_0, Q4_0 or Q4_K weight of 2048 or 4096 columns and a multiple of eight
 * (four) rows takes two launches instead of three: the projection's workgroups keep the largest
 * logit they store and its row, and the second launch folds those thousand candidates instead of
 * reading the logits back.  Any other weight the single-token kernels take is the two calls, made
 * here.
 */
int jl_gemv_argmax(jl_context *ctx, const jl_weight *w, const float *x, const float *rms_weights,
                   const float *rms_scale, float eps, float *out, int32_t *index);

/*
 * jl_argmax for callers that cannot allocate device memory: code under HIP graph capture, tight
 * serving loops, harnesses that forbid hipMalloc.  It has no counterpart in the reference.  The
 * candidates that the first launch hands to the second -- one (value, index) cell per scanning
 * workgroup, 1 KiB -- live in a device array that is part of the library's code object, so neither
 * this call nor anything it relies on (hipMalloc, hipFree, an allocating library routine) allocates;
 * jl_argmax keeps them in memory that jl_context_create allocated.  The result is jl_argmax's.
 *   - at most JL_ARGMAX_STATIC_MAX_VALUES values; more is JL_ERR_INVALID, use jl_argmax.
 *   - every call on one GPU shares that GPU's array, whatever the context or stream: calls that
 *     overlap on one GPU race.  Calls ordered on one stream do not; a call reads no cell it has
 *     not written itself, so nothing needs clearing between calls.
 *   - the array's address is looked up per device by jl_context_create (devices 0..63).
 */
#define JL_ARGMAX_STATIC_MAX_VALUES ((int64_t)1 << 24)
int jl_argmax_static(jl_context *ctx, const float *values, int64_t n, int32_t *index);

/* ---- packed-activation ("dp4a") decode: faster, looser -------------------------------------- */
/*
 * The reference's optional packed-integer decode path (QuantizedProjections.packed(),
 * J/backend/tornado/layers/QuantizedProjections.java:110-190,257-346): the activation is quantised
 * once to Q8 blocks and every projection of it is a sum of exact int32 block dot products times
 * the two block scales.  It does NOT meet the 1e-3 bound of the entry points above -- the
 * activation keeps 8 bits -- and is held to the reference's own looser envelope for this path
 * (src/test/.../golden/CpuGpuParity.java:115-116); what it is held to tightly is the reference's
 * packed arithmetic itself.  Q8_0, Q4_0 and Q4_K weights; row lengths that are multiples of 64 up
 * to 16384 (8192 for gate/up); `quants` 16-byte aligned, `scales` and `sums` 8-byte aligned.
 *
 * jl_quantize_q8: quantizeActivationQ8Blocks (TransformerComputeKernelsQ4_0.java:287-341).  Per
 * block of 32: inverse = 127 / max|x| (0 for a block of zeros), q = (int)(x * inverse +- 0.5)
 * clamped to +-127, scales[b] = max|x| / 127, sums[b] = sum of the block's q.  n must be a multiple
 * of 32; quants holds n bytes in element order, scales and sums n / 32 entries.
 */
int jl_quantize_q8(jl_context *ctx, const float *x, int64_t n, int8_t *quants, float *scales, int32_t *sums);
/*
 * The RMS-norm apply and the quantisation in one launch: xb[i] = rms_weights[i] * (rms_scale[0] * x[i])
 * (both products rounded to fp32; rms_scale is the device scalar jl_rms_scale leaves) is written --
 * non-packed readers still need it -- and quantised as above.  rmsApplyAndQuantizeActivationQ8Blocks
 * (TransformerComputeKernelsQ4_0.java:374-432), dispatched by QuantizedProjections.rmsApply
 * (QuantizedProjections.java:117-121) before the packed projections of a layer.
 */
int jl_rms_quantize_q8(jl_context *ctx, const float *x, const float *rms_weights, const float *rms_scale,
                       int64_t n, float *xb, int8_t *quants, float *scales, int32_t *sums);
/*
 * out (+)= W . x~ with x~ the quantised activation: matrixVectorGenericQ8_0DP4A / ...WithResidual
 * (TransformerComputeKernelsQ8_0DP4A.java:71-97,245-268), ...Q4_0DP4A (TransformerComputeKernelsQ4_0.java:
 * 466-524,773+), ...Q4_KDP4A (TransformerComputeKernelsQ4_K.java:446-515).  Per block:
 * Q8_0 (dW sX) dot; Q4_0 (dW sX) (dot - 8 sum); Q4_K d (sc sX dot) - dmin (m sX sum).
 */
int jl_gemv_q8(jl_context *ctx, const jl_weight *w, const int8_t *quants, const float *scales,
               const int32_t *sums, float *out, int epilogue);
/* fusedQKVMatmulQ8_0DP4A (TransformerComputeKernelsQ8_0DP4A.java:129-176) and its siblings. */
int jl_gemv_qkv_q8(jl_context *ctx, const jl_weight *wq, const jl_weight *wk, const jl_weight *wv,
                   const int8_t *quants, const float *scales, const int32_t *sums, float *q, float *k, float *v);
/* fusedFFNGateUpSiLUQ8_0DP4A (:295-346), ...Q4_0DP4A (TransformerComputeKernelsQ4_0.java:859-950),
 * ...Q4_KDP4A (TransformerComputeKernelsQ4_K.java:520-574). */
int jl_gemv_gate_up_q8(jl_context *ctx, const jl_weight *w1, const jl_weight *w3, const int8_t *quants,
                       const float *scales, const int32_t *sums, float *hb);

/* ---- batched decode and batched prefill: `batch` activation rows ---------------------------- */

/*
 * Bytes of scratch jl_gemm needs (Implementation.needs,
 * J/backend/tornado/ops/Implementation.java:31-36: sized before anything is allocated, so a
 * memory preflight equals what the call uses).  `max_rows` is the largest `batch`, `cols` the
 * largest row length, `out_cols` the largest number of output columns one call produces (a gate/up
 * pair counts both weights' rows), `math` a jl_gemm_math.  The scratch holds the fp16 copy of the
 * activations, one scale per row, and a third region of about 2.1 bytes per weight of the largest
 * call that a call uses for one of two things: the partial sums of calls that cut K across
 * workgroups (calls whose tile grid would leave compute units idle), or -- calls of 512 rows and
 * more, the reference's dequantize-then-gemmMMA prefill shape -- an fp16 copy of the call's
 * weights, decoded afresh by every such call and dead after it (beside it the partial sums of
 * narrow projections, which also calls of 128 rows and more over a kept copy use: the size counts
 * them from max_rows = 128).  A smaller workspace that still
 * holds the first two is accepted; such calls simply keep to one pass and do not cut K.  Calls of
 * at most 64 rows -- and calls of up to 511 rows whose weights are small enough that streaming
 * them once per 32 rows beats the tiled kernels -- read X directly and use only the partial sums.
 */
size_t jl_gemm_workspace_bytes(int64_t max_rows, int64_t cols, int64_t out_cols, int math);

/*
 * C[b][col_offset + j] (op)= sum_k X[b][k] * W_i[j][k] for the `count` weights laid side by
 * side (C = A.[W0|W1|...]^T, FP16Projections / DecodedMatMul.project :93-109), over the first
 * `active_rows` of `batch` rows; rows past active_rows are left exactly as they were
 * (QuantizedBatchProjections.projection :76-309, matrixVectorTiledBatchQ4_0/Q4_K's activeRows).
 *   X    [batch x cols] fp32 row-major          C  fp32, row stride `ldo` floats
 *   epilogue JL_STORE / JL_RESIDUAL, or JL_SWIGLU with count == 2 (gate, up):
 *            C[b][col_offset + j] = SiLU(X_b.W0_j) * (X_b.W1_j)
 *   math     a jl_gemm_math.  JL_MATH_INT8 (Q8_0 and Q4_0 weights; other types JL_ERR_UNSUPPORTED) is
 *            the block-scaled int8 arithmetic of Int8GemmKernels.java:17-23 -- activations quantised
 *            per 32-block inside the call (quantizeActivationsQ8Warp :96-129), each block's dot
 *            product exact in int32, acc = fma((float) dot * dA, dW, acc) over the blocks in k order,
 *            SwiGLU as (g / (1 + exp(-g))) * u in fp32 -- reproduced step by step, K never cut: the
 *            fp32 results of JL_STORE / JL_RESIDUAL are those of that arithmetic bit for bit.  It
 *            reads the raw blocks where they lie (gemmInt8Q8_0 :651-676) and takes row lengths that
 *            are multiples of 64.  An opt-in mode: an activation carries 7 bits, so against the
 *            fp32 CPU path it is looser than JL_MATH_F16 (every output within sum over the blocks
 *            of (dA / 2) * sum |w|).
 * JL_MATH_F16: the row length must be a multiple of 64 columns, else JL_ERR_UNSUPPORTED (rows of
 * whole 256-column blocks have kernels for every row count; others -- 896 columns -- are decoded to
 * fp16 in the workspace on every call, as the types without a fused kernel are).  The
 * weights of a call may differ in type (a "Q4_K_M" file's q | k | v with v in Q6_K; a gate and an up
 * weight of different types): each is then decoded to fp16 by its own type and one fp16 GEMM
 * multiplies them, as the reference's prefill projections do (FP16Projections.project,
 * J/backend/tornado/layers/FP16Projections.java:250-330: one decode task per weight, chosen by its
 * dataType()); such a call needs the workspace jl_gemm_workspace_bytes gives for its `out_cols` (or
 * a resident buffer) whatever its row count.  JL_MATH_INT8 multiplies the raw blocks and refuses
 * mixed types.
 * This is Int8GemmKernels.gemmInt8Q8_0's contract (:651-676: epilogue, rowsHolder, ldo,
 * colOffset) and gemmMMAQ8's, behind one call.
 */
int jl_gemm(jl_context *ctx, const jl_weight *const *weights, int count, const float *X, float *C,
            int64_t batch, int64_t active_rows, int64_t ldo, int64_t col_offset, int epilogue,
            int math, void *workspace, size_t workspace_bytes);

/*
 * jl_gemm with a resident fp16 copy of the call's weights: the reference's "residency choice" for
 * the batched prefill (dequantize*ToFP16Once, TransformerBatchPrefillKernels.java:2336-2366: "the
 * copy outlives the chunk, so it is decoded on the first one only"; BatchPrefillWorkspace).  Calls
 * that decode their weights to fp16 (512 rows and more with enough output columns, and every Q6_K /
 * Q5_K call) put the copy into `resident` instead of the workspace, and skip the decode when
 * `*resident_state` says the buffer already holds what they need.  The caller owns one buffer of
 * jl_gemm_resident_bytes(weights, count) bytes (2 per weight) and one int32 per set of weights it
 * passes together, zeroes the int before the first call and whenever the weights' contents change,
 * and never shares a buffer between different sets.  The state records the layout of the copy, not
 * whose weights it holds: reset *resident_state to 0 whenever the set of weights behind the buffer
 * changes -- also when a weight is freed and another one is uploaded in its place, even if the new
 * jl_weight comes back at the old address.  Calls that do not decode ignore both.  Results are the
 * same as jl_gemm's, bit for bit -- except that calls of 128 .. 511 rows may run the plain fp16 GEMM
 * over a kept copy where jl_gemm, which would have to decode first, runs a kernel that decodes as it
 * goes: the same products of the same fp16 operands, added in fp32 in another order.
 */
size_t jl_gemm_resident_bytes(const jl_weight *const *weights, int count);
int jl_gemm_resident(jl_context *ctx, const jl_weight *const *weights, int count, const float *X, float *C,
                     int64_t batch, int64_t active_rows, int64_t ldo, int64_t col_offset, int epilogue,
                     int math, void *workspace, size_t workspace_bytes, void *resident,
                     size_t resident_bytes, int32_t *resident_state);

/*
 * jl_gemm / jl_gemm_resident over activations that are already fp16 -- what the reference's prefill
 * plugin is handed: DecodedMatMul.project (J/backend/tornado/ops/DecodedMatMul.java:100-109) passes
 * the step's input as a HalfFloatArray and its output as a FloatArray, gemmMMA / gemmMMAQ8 take
 * `HalfFloatArray A` (TransformerBatchPrefillKernels.java:917-924, 2397+), and the producers write
 * fp16 themselves (batchedRmsApplyFP16 :59-72, batchedDecodeAttentionFP16Out :1633+,
 * batchedFFNSwiGLUFP16Packed :2183-2199).
 *   X    [batch x cols] IEEE binary16 row-major, 16-byte aligned, multiplied as it is (jl_gemm
 *        first rescales every fp32 row by a power of two; there is nothing to rescale here, so a
 *        row whose products leave fp16's range is the producer's to avoid, as in the reference).
 *        Calls that read whole 256-row tiles take X in place when `batch` covers the last tile,
 *        otherwise the active rows are copied into the workspace first.  Calls of at most 64 active
 *        rows -- a short prompt, the tail of a chunked one -- run jl_gemm's weight-streaming kernel,
 *        which reads X where it lies and brings every row into range by a power of two as it does
 *        for fp32 rows (exact, undone on the results).
 *   C    fp32 as in jl_gemm; with c_fp16 != 0 -- JL_SWIGLU only, the feed-forward hidden vector
 *        batchedFFNSwiGLUFP16Packed writes -- binary16, `ldo` and `col_offset` counting fp16 values
 *        and every result rounded once from its fp32 value.
 *   resident / resident_state: as in jl_gemm_resident, or both null for jl_gemm's behaviour.
 * The workspace is sized by jl_gemm_workspace_bytes as for jl_gemm.  On inputs that fp16 holds
 * exactly and whose rows jl_gemm's rescaling does not push below fp16's normal range the fp32
 * results equal, bit for bit, those of jl_gemm (resident null) or jl_gemm_resident (the same
 * resident buffer) on the widened inputs.
 */
int jl_gemm_xf16(jl_context *ctx, const jl_weight *const *weights, int count, const uint16_t *X, void *C,
                 int c_fp16, int64_t batch, int64_t active_rows, int64_t ldo, int64_t col_offset, int epilogue,
                 void *workspace, size_t workspace_bytes, void *resident, size_t resident_bytes,
                 int32_t *resident_state);

/*
 * The producer of those fp16 activations: the batched prefill's RMS normalisation, reduction and
 * apply in one launch.  batchedRmsReduceParallel (TransformerBatchPrefillKernels.java:1480-1510)
 * in its own summation order -- work item t of 256 adds the squares of elements t, t + 256, ...,
 * the partial sums fold as a binary tree, scales[b] = 1 / sqrt(sum / n + eps) in fp32 -- then
 * batchedRmsApplyFP16 (:59-72): out[b][i] = fp16(rms_weights[i] * scales[b] * X[b][i]), products
 * left to right in fp32, one rounding to fp16.  X [rows x n] fp32, out [rows x n] binary16;
 * `scales` ([rows]) may be null.  With `delta` ([rows x n], else null) the pending residual add
 * comes first -- batchedRmsReduceFusedResidual (:1519-1551): X[b][i] += delta[b][i] is written
 * back and sums and outputs are those of the updated row; without it X is only read.
 */
int jl_rms_apply_xf16(jl_context *ctx, float *X, const float *delta, const float *rms_weights, float eps,
                      int64_t rows, int64_t n, float *scales, uint16_t *out);

/* ---- GGUF files: the caller either side of jl_weight_upload --------------------------------- */

/*
 * Parses a GGUF file's header, metadata and tensor infos and keeps the file mapped read-only
 * (GGUF.loadGGUFMetadata, J/format/GGUF.java:40-115; versions 2 and 3, general.alignment or 32).
 * A file the reference refuses is refused with the same words: "unsupported header.magic ...",
 * "unsupported header.version ...", "Model file not found: ...".  Host work only; needs no GPU.
 */
typedef struct jl_gguf jl_gguf;
int jl_gguf_open(const char *path, jl_gguf **out);
int jl_gguf_close(jl_gguf *g);
int jl_gguf_version(const jl_gguf *g);
int jl_gguf_alignment(const jl_gguf *g);
int64_t jl_gguf_data_offset(const jl_gguf *g);   /* file offset of the tensor-data section (:71-96) */
int64_t jl_gguf_tensor_count(const jl_gguf *g);
int64_t jl_gguf_metadata_count(const jl_gguf *g);

/*
 * Tensor `index` in file order, or by name (jl_gguf_find: index, -1 if absent): GGUFTensorInfo
 * (J/format/GGUF.java:297-322, 520).  `dims` are in GGUF ne order (dims[0] = row length), unused
 * ones 1; `file_offset` is absolute; `bytes` follows the block geometry of J/format/GGMLType.java:5-54
 * and is -1 for a type the reference cannot read either.  `name` stays valid until jl_gguf_close.
 */
int64_t jl_gguf_find(const jl_gguf *g, const char *name);
int jl_gguf_tensor_info(const jl_gguf *g, int64_t index, const char **name, int *ggml_type, int *n_dims,
                        int64_t dims[4], int64_t *file_offset, int64_t *bytes);

/*
 * Metadata by key (GGUF.readHeader / readMetadataValueOfType, :365-474): integers and booleans as
 * int64, floats as double, strings by pointer (valid until jl_gguf_close); of an array only the
 * element type (gguf_metadata_value_type) and the count are kept.  A missing key or a value of
 * another kind is JL_ERR_INVALID.
 */
int jl_gguf_metadata_int(const jl_gguf *g, const char *key, int64_t *value);
int jl_gguf_metadata_float(const jl_gguf *g, const char *key, double *value);
int jl_gguf_metadata_string(const jl_gguf *g, const char *key, const char **value, int64_t *length);
int jl_gguf_metadata_array(const jl_gguf *g, const char *key, int *element_type, int64_t *count);

/*
 * jl_weight_upload of a two-dimensional Q8_0 / Q4_0 / Q4_K / Q5_K / Q6_K tensor straight from the mapped file
 * (ModelLoader.loadTornadoTensorNative, J/model/loader/ModelLoader.java:246-290, without the
 * 16-byte array header the reference's segments carry, GGUF.java:214-268).  Another type is
 * JL_ERR_UNSUPPORTED naming it; a tensor that runs past the end of the file is refused (:236-247).
 */
int jl_gguf_upload(jl_context *ctx, const jl_gguf *g, const char *name, jl_weight **out);

#ifdef __cplusplus
}
#endif
#endif
