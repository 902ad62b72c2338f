// C-ABI entry points of libjitllm_hip.so: context, device buffers, weights, argument checks.
// The kernels live in jl_dequant.hip, jl_gemv.hip and jl_gemm.hip.
#include <stdarg.h>
#include <string.h>

#include <new>

#include "jl_internal.h"

static thread_local char g_error[512] = "";

int jl_fail(int status, const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_error, sizeof g_error, fmt, ap);
    va_end(ap);
    return status;
}

extern "C" {

int jl_abi_version(void) { return JL_ABI_VERSION; }

const char *jl_last_error(void) { return g_error; }

static void context_release(jl_context *ctx) {
    for (int i = 0; i < 2; i++)
        if (ctx->bounce_done[i]) (void)hipEventDestroy(ctx->bounce_done[i]);
    if (ctx->bounce) (void)hipHostFree(ctx->bounce);
    if (ctx->scratch) (void)hipFree(ctx->scratch);
    if (ctx->arrivals) (void)hipFree(ctx->arrivals);
    if (ctx->owns_stream) (void)hipStreamDestroy(ctx->stream);
    delete ctx;
}

static int context_create(int device, hipStream_t borrowed, bool borrow, jl_context **out) {
    JL_REQUIRE(out != nullptr, "jl_context_create: out is null");
    *out = nullptr;
    int count = 0;
    JL_HIP(hipGetDeviceCount(&count));
    JL_REQUIRE(device >= 0 && device < count, "jl_context_create: device %d of %d", device, count);
    JL_HIP(hipSetDevice(device));
    hipDeviceProp_t prop;
    JL_HIP(hipGetDeviceProperties(&prop, device));
    if (strncmp(prop.gcnArchName, "gfx950", 6) != 0) {
        return jl_fail(JL_ERR_UNSUPPORTED,
                       "device %d is %s; this library carries gfx950 (MI355X) code only", device,
                       prop.gcnArchName);
    }
    {
        const int st = jl_static_scratch_init(device);   // `device` is current
        if (st != JL_OK) return st;
    }
    jl_context *ctx = new (std::nothrow) jl_context();
    JL_REQUIRE(ctx != nullptr, "jl_context_create: host allocation failed");
    ctx->device = device;
    ctx->compute_units = prop.multiProcessorCount;
    snprintf(ctx->name, sizeof ctx->name, "%s", prop.name[0] ? prop.name : prop.gcnArchName);
    if (borrow) {
        ctx->stream = borrowed;
        ctx->owns_stream = false;
    } else {
        hipError_t e = hipStreamCreateWithFlags(&ctx->stream, hipStreamNonBlocking);
        if (e != hipSuccess) {
            delete ctx;
            return jl_fail(JL_ERR_HIP, "hipStreamCreateWithFlags failed: %s", hipGetErrorString(e));
        }
        ctx->owns_stream = true;
    }
    hipError_t e = hipMalloc(&ctx->scratch, JL_CONTEXT_SCRATCH_BYTES);   // written before it is read
    if (e == hipSuccess) e = hipMalloc((void **)&ctx->arrivals, JL_CONTEXT_ARRIVALS * sizeof(uint32_t));
    // (on the context's own stream, which does not wait for the default stream, and waited for)
    if (e == hipSuccess) e = hipMemsetAsync(ctx->arrivals, 0, JL_CONTEXT_ARRIVALS * sizeof(uint32_t), ctx->stream);
    if (e == hipSuccess) e = hipStreamSynchronize(ctx->stream);
    if (e == hipSuccess) e = hipHostMalloc((void **)&ctx->bounce, 2 * (size_t)JL_BOUNCE_HALF_BYTES, hipHostMallocDefault);
    for (int i = 0; i < 2 && e == hipSuccess; i++) e = hipEventCreateWithFlags(&ctx->bounce_done[i], hipEventDisableTiming);
    if (e != hipSuccess) {
        context_release(ctx);
        return jl_fail(JL_ERR_OOM, "jl_context_create: scratch / staging allocation failed: %s", hipGetErrorString(e));
    }
    *out = ctx;
    return JL_OK;
}

int jl_context_create(int device, jl_context **out) {
    return context_create(device, nullptr, false, out);
}

int jl_context_create_on_stream(int device, void *hip_stream, jl_context **out) {
    return context_create(device, (hipStream_t)hip_stream, true, out);
}

int jl_context_destroy(jl_context *ctx) {
    if (!ctx) return JL_OK;
    (void)hipSetDevice(ctx->device);
    (void)hipStreamSynchronize(ctx->stream);
    context_release(ctx);
    return JL_OK;
}

int jl_sync(jl_context *ctx) {
    JL_REQUIRE(ctx != nullptr, "jl_sync: context is null");
    JL_HIP(hipStreamSynchronize(ctx->stream));
    return JL_OK;
}

void *jl_context_stream(jl_context *ctx) { return ctx ? (void *)ctx->stream : nullptr; }

int jl_context_set_split_k(jl_context *ctx, int enabled) {
    JL_REQUIRE(ctx != nullptr, "jl_context_set_split_k: context is null");
    ctx->split_k = enabled != 0;
    return JL_OK;
}

int jl_device_info(jl_context *ctx, int *compute_units, char *name, size_t name_bytes) {
    JL_REQUIRE(ctx != nullptr, "jl_device_info: context is null");
    if (compute_units) *compute_units = ctx->compute_units;
    if (name && name_bytes) snprintf(name, name_bytes, "%s", ctx->name);
    return JL_OK;
}

int jl_malloc(jl_context *ctx, size_t bytes, void **device_ptr) {
    JL_REQUIRE(ctx && device_ptr, "jl_malloc: null argument");
    *device_ptr = nullptr;
    JL_HIP(hipSetDevice(ctx->device));
    hipError_t e = hipMalloc(device_ptr, bytes ? bytes : 16);
    if (e != hipSuccess) {
        return jl_fail(JL_ERR_OOM, "device allocation of %zu bytes failed: %s", bytes,
                       hipGetErrorString(e));
    }
    return JL_OK;
}

int jl_free(jl_context *ctx, void *device_ptr) {
    JL_REQUIRE(ctx != nullptr, "jl_free: context is null");
    if (!device_ptr) return JL_OK;
    JL_HIP(hipStreamSynchronize(ctx->stream));
    JL_HIP(hipFree(device_ptr));
    return JL_OK;
}

// Host memory handed to these two is the caller's, pageable as a rule (a Java heap segment, a numpy
// array, a mapped file).  It is copied through the context's pinned staging halves in turn, so the
// device only ever runs DMA transfers against pinned memory and the runtime's own handling of
// pageable pointers (staging of its own, or host writes straight into device memory) is not used.
int jl_upload(jl_context *ctx, void *device_dst, const void *host_src, size_t bytes) {
    JL_REQUIRE(ctx && (bytes == 0 || (device_dst && host_src)), "jl_upload: null argument");
    if (!bytes) return JL_OK;
    JL_HIP(hipSetDevice(ctx->device));
    const uint8_t *src = (const uint8_t *)host_src;
    uint8_t *dst = (uint8_t *)device_dst;
    int half = 0;
    bool used[2] = {false, false};
    for (size_t done = 0; done < bytes; half ^= 1) {
        const size_t n = bytes - done < JL_BOUNCE_HALF_BYTES ? bytes - done : (size_t)JL_BOUNCE_HALF_BYTES;
        uint8_t *stage = ctx->bounce + (size_t)half * JL_BOUNCE_HALF_BYTES;
        if (used[half]) JL_HIP(hipEventSynchronize(ctx->bounce_done[half]));   // its last transfer has left it
        memcpy(stage, src + done, n);
        JL_HIP(hipMemcpyAsync(dst + done, stage, n, hipMemcpyHostToDevice, ctx->stream));
        JL_HIP(hipEventRecord(ctx->bounce_done[half], ctx->stream));
        used[half] = true;
        done += n;
    }
    JL_HIP(hipStreamSynchronize(ctx->stream));
    return JL_OK;
}

int jl_download(jl_context *ctx, void *host_dst, const void *device_src, size_t bytes) {
    JL_REQUIRE(ctx && (bytes == 0 || (host_dst && device_src)), "jl_download: null argument");
    if (!bytes) return JL_OK;
    JL_HIP(hipSetDevice(ctx->device));
    uint8_t *dst = (uint8_t *)host_dst;
    const uint8_t *src = (const uint8_t *)device_src;
    // chunk i + 1 is on its way into the other half while chunk i is copied out to the caller
    size_t issued = 0, copied = 0;
    size_t len[2] = {0, 0};
    int half = 0;
    auto issue = [&](int h) -> hipError_t {
        len[h] = bytes - issued < JL_BOUNCE_HALF_BYTES ? bytes - issued : (size_t)JL_BOUNCE_HALF_BYTES;
        hipError_t e = hipMemcpyAsync(ctx->bounce + (size_t)h * JL_BOUNCE_HALF_BYTES, src + issued, len[h],
                                      hipMemcpyDeviceToHost, ctx->stream);
        if (e == hipSuccess) e = hipEventRecord(ctx->bounce_done[h], ctx->stream);
        issued += len[h];
        return e;
    };
    JL_HIP(issue(0));
    while (copied < bytes) {
        if (issued < bytes) JL_HIP(issue(half ^ 1));
        JL_HIP(hipEventSynchronize(ctx->bounce_done[half]));
        memcpy(dst + copied, ctx->bounce + (size_t)half * JL_BOUNCE_HALF_BYTES, len[half]);
        copied += len[half];
        half ^= 1;
    }
    return JL_OK;
}

int jl_fill_f32(jl_context *ctx, float *device_dst, float value, size_t count) {
    JL_REQUIRE(ctx && (count == 0 || device_dst), "jl_fill_f32: null argument");
    if (!count) return JL_OK;
    return jl_launch_fill(ctx, device_dst, value, count);
}

static int weight_check(const char *who, int type, int64_t rows, int64_t cols) {
    if (jl_block_elems(type) == 0) {
        return jl_fail(JL_ERR_UNSUPPORTED, "%s: no projection kernel for a ggml type %d weight", who,
                       type);
    }
    JL_REQUIRE(rows > 0 && cols > 0, "%s: shape %lld x %lld", who, (long long)rows, (long long)cols);
    JL_REQUIRE(cols % jl_block_elems(type) == 0,
               "%s: row length %lld is not a whole number of %s blocks (%d)", who, (long long)cols,
               jl_type_name(type), jl_block_elems(type));
    JL_REQUIRE(rows <= INT32_MAX && cols <= INT32_MAX, "%s: shape exceeds 2^31", who);
    return JL_OK;
}

int jl_weight_upload(jl_context *ctx, int ggml_type, const void *host_blocks, int64_t rows,
                     int64_t cols, jl_weight **out) {
    JL_REQUIRE(ctx && host_blocks && out, "jl_weight_upload: null argument");
    *out = nullptr;
    int st = weight_check("jl_weight_upload", ggml_type, rows, cols);
    if (st != JL_OK) return st;
    int64_t bytes = rows * (cols / jl_block_elems(ggml_type)) * jl_block_bytes(ggml_type);
    void *dev = nullptr;
    st = jl_malloc(ctx, (size_t)bytes, &dev);
    if (st != JL_OK) return st;
    st = jl_upload(ctx, dev, host_blocks, (size_t)bytes);
    if (st != JL_OK) {
        (void)hipFree(dev);
        return st;
    }
    jl_weight *w = new (std::nothrow) jl_weight();
    if (!w) {
        (void)hipFree(dev);
        return jl_fail(JL_ERR_INVALID, "jl_weight_upload: host allocation failed");
    }
    *w = jl_weight{ctx, ggml_type, rows, cols, bytes, (const uint8_t *)dev, true};
    *out = w;
    return JL_OK;
}

int jl_weight_wrap(jl_context *ctx, int ggml_type, const void *device_blocks, int64_t rows,
                   int64_t cols, jl_weight **out) {
    JL_REQUIRE(ctx && device_blocks && out, "jl_weight_wrap: null argument");
    *out = nullptr;
    int st = weight_check("jl_weight_wrap", ggml_type, rows, cols);
    if (st != JL_OK) return st;
    JL_REQUIRE(((uintptr_t)device_blocks & 15) == 0,
               "jl_weight_wrap: blocks must be 16-byte aligned in device memory");
    int64_t bytes = rows * (cols / jl_block_elems(ggml_type)) * jl_block_bytes(ggml_type);
    jl_weight *w = new (std::nothrow) jl_weight();
    JL_REQUIRE(w != nullptr, "jl_weight_wrap: host allocation failed");
    *w = jl_weight{ctx, ggml_type, rows, cols, bytes, (const uint8_t *)device_blocks, false};
    *out = w;
    return JL_OK;
}

int jl_weight_free(jl_weight *w) {
    if (!w) return JL_OK;
    int st = JL_OK;
    if (w->owns_blocks) st = jl_free(w->ctx, (void *)w->blocks);
    delete w;
    return st;
}

int jl_weight_info(const jl_weight *w, int *ggml_type, int64_t *rows, int64_t *cols,
                   int64_t *bytes) {
    JL_REQUIRE(w != nullptr, "jl_weight_info: weight is null");
    if (ggml_type) *ggml_type = w->type;
    if (rows) *rows = w->rows;
    if (cols) *cols = w->cols;
    if (bytes) *bytes = w->bytes;
    return JL_OK;
}

const void *jl_weight_blocks(const jl_weight *w) { return w ? w->blocks : nullptr; }

int jl_dequant_f32(jl_context *ctx, const jl_weight *w, float *out) {
    JL_REQUIRE(ctx && w && out, "jl_dequant_f32: null argument");
    return jl_launch_dequant(ctx, w, out);
}

int jl_gemv(jl_context *ctx, const jl_weight *w, const float *x, float *out, int epilogue) {
    JL_REQUIRE(ctx && w && x && out, "jl_gemv: null argument");
    JL_REQUIRE(epilogue == JL_STORE || epilogue == JL_RESIDUAL,
               "jl_gemv: epilogue %d (JL_STORE or JL_RESIDUAL)", epilogue);
    return jl_launch_gemv(ctx, &w, 1, &out, nullptr, x, epilogue, nullptr);
}

int jl_gemv_qkv(jl_context *ctx, const jl_weight *wq, const jl_weight *wk, const jl_weight *wv,
                const float *x, float *q, float *k, float *v) {
    JL_REQUIRE(ctx && wq && wk && wv && x && q && k && v, "jl_gemv_qkv: null argument");
    if (wq->type != wk->type || wq->type != wv->type) {
        return jl_fail(JL_ERR_UNSUPPORTED,
                       "jl_gemv_qkv: no fused q|k|v kernel for mixed weights %s/%s/%s",
                       jl_type_name(wq->type), jl_type_name(wk->type), jl_type_name(wv->type));
    }
    JL_REQUIRE(wq->cols == wk->cols && wq->cols == wv->cols,
               "jl_gemv_qkv: row lengths differ (%lld, %lld, %lld)", (long long)wq->cols,
               (long long)wk->cols, (long long)wv->cols);
    const jl_weight *ws[3] = {wq, wk, wv};
    float *outs[3] = {q, k, v};
    return jl_launch_gemv(ctx, ws, 3, outs, nullptr, x, JL_STORE, nullptr);
}

int jl_gemv_gate_up(jl_context *ctx, const jl_weight *w1, const jl_weight *w3, const float *x,
                    float *hb) {
    JL_REQUIRE(ctx && w1 && w3 && x && hb, "jl_gemv_gate_up: null argument");
    if (w1->type != w3->type) {
        return jl_fail(JL_ERR_UNSUPPORTED,
                       "jl_gemv_gate_up: no fused gate/up kernel for a %s gate and a %s up weight",
                       jl_type_name(w1->type), jl_type_name(w3->type));
    }
    JL_REQUIRE(w1->rows == w3->rows && w1->cols == w3->cols,
               "jl_gemv_gate_up: gate is %lld x %lld, up is %lld x %lld", (long long)w1->rows,
               (long long)w1->cols, (long long)w3->rows, (long long)w3->cols);
    return jl_launch_gemv(ctx, &w1, 1, &hb, w3, x, JL_SWIGLU, nullptr);
}

int jl_rms_scale(jl_context *ctx, const float *x, int64_t n, float eps, float *scale) {
    JL_REQUIRE(ctx && x && scale && n > 0, "jl_rms_scale: bad argument");
    return jl_launch_rms_scale(ctx, x, n, eps, scale);
}

int jl_rms_apply(jl_context *ctx, const float *x, const float *rms_weights, const float *rms_scale, int64_t n,
                 float *xb) {
    JL_REQUIRE(ctx && x && rms_weights && rms_scale && xb && n > 0 && n <= (int64_t)UINT32_MAX * 256,
               "jl_rms_apply: bad argument");
    return jl_launch_rms_apply(ctx, x, rms_weights, rms_scale, n, xb);
}

int jl_gemv_rms(jl_context *ctx, const jl_weight *w, const float *x, const float *rms_weights,
                const float *rms_scale, float eps, float *out, int epilogue) {
    JL_REQUIRE(ctx && w && x && rms_weights && out, "jl_gemv_rms: null argument");
    JL_REQUIRE(epilogue == JL_STORE || epilogue == JL_RESIDUAL,
               "jl_gemv_rms: epilogue %d (JL_STORE or JL_RESIDUAL)", epilogue);
    const jl_rms rms{rms_weights, rms_scale, eps};
    return jl_launch_gemv(ctx, &w, 1, &out, nullptr, x, epilogue, &rms);
}

int jl_gemv_qkv_rms(jl_context *ctx, const jl_weight *wq, const jl_weight *wk, const jl_weight *wv,
                    const float *x, const float *rms_weights, const float *rms_scale, float eps,
                    float *q, float *k, float *v) {
    JL_REQUIRE(ctx && wq && wk && wv && x && rms_weights && q && k && v,
               "jl_gemv_qkv_rms: null argument");
    if (wq->type != wk->type || wq->type != wv->type) {
        return jl_fail(JL_ERR_UNSUPPORTED,
                       "jl_gemv_qkv_rms: no fused q|k|v kernel for mixed weights %s/%s/%s",
                       jl_type_name(wq->type), jl_type_name(wk->type), jl_type_name(wv->type));
    }
    JL_REQUIRE(wq->cols == wk->cols && wq->cols == wv->cols,
               "jl_gemv_qkv_rms: row lengths differ (%lld, %lld, %lld)", (long long)wq->cols,
               (long long)wk->cols, (long long)wv->cols);
    const jl_weight *ws[3] = {wq, wk, wv};
    float *outs[3] = {q, k, v};
    const jl_rms rms{rms_weights, rms_scale, eps};
    return jl_launch_gemv(ctx, ws, 3, outs, nullptr, x, JL_STORE, &rms);
}

int jl_gemv_gate_up_rms(jl_context *ctx, const jl_weight *w1, const jl_weight *w3, const float *x,
                        const float *rms_weights, float eps, float *hb) {
    JL_REQUIRE(ctx && w1 && w3 && x && rms_weights && hb, "jl_gemv_gate_up_rms: null argument");
    if (w1->type != w3->type) {
        return jl_fail(JL_ERR_UNSUPPORTED,
                       "jl_gemv_gate_up_rms: no fused gate/up kernel for a %s gate and a %s up weight",
                       jl_type_name(w1->type), jl_type_name(w3->type));
    }
    JL_REQUIRE(w1->rows == w3->rows && w1->cols == w3->cols,
               "jl_gemv_gate_up_rms: gate is %lld x %lld, up is %lld x %lld", (long long)w1->rows,
               (long long)w1->cols, (long long)w3->rows, (long long)w3->cols);
    const jl_rms rms{rms_weights, nullptr, eps};
    return jl_launch_gemv(ctx, &w1, 1, &hb, w3, x, JL_SWIGLU, &rms);
}

int jl_quantize_q8(jl_context *ctx, const float *x, int64_t n, int8_t *quants, float *scales, int32_t *sums) {
    JL_REQUIRE(ctx && x && quants && scales && sums, "jl_quantize_q8: null argument");
    JL_REQUIRE(n > 0 && n % 32 == 0, "jl_quantize_q8: %lld activations are not a whole number of blocks of 32",
               (long long)n);
    return jl_launch_quantize_q8(ctx, x, nullptr, nullptr, nullptr, n, quants, scales, sums);
}

int jl_rms_quantize_q8(jl_context *ctx, const float *x, const float *rms_weights, const float *rms_scale,
                       int64_t n, float *xb, int8_t *quants, float *scales, int32_t *sums) {
    JL_REQUIRE(ctx && x && rms_weights && rms_scale && xb && quants && scales && sums,
               "jl_rms_quantize_q8: null argument");
    JL_REQUIRE(n > 0 && n % 32 == 0, "jl_rms_quantize_q8: %lld activations are not a whole number of blocks of 32",
               (long long)n);
    return jl_launch_quantize_q8(ctx, x, rms_weights, rms_scale, xb, n, quants, scales, sums);
}

int jl_gemv_q8(jl_context *ctx, const jl_weight *w, const int8_t *quants, const float *scales,
               const int32_t *sums, float *out, int epilogue) {
    JL_REQUIRE(ctx && w && quants && scales && sums && out, "jl_gemv_q8: null argument");
    JL_REQUIRE(epilogue == JL_STORE || epilogue == JL_RESIDUAL,
               "jl_gemv_q8: epilogue %d (JL_STORE or JL_RESIDUAL)", epilogue);
    const jl_q8x xq{quants, scales, sums};
    return jl_launch_gemv(ctx, &w, 1, &out, nullptr, nullptr, epilogue, nullptr, &xq);
}

int jl_gemv_qkv_q8(jl_context *ctx, const jl_weight *wq, const jl_weight *wk, const jl_weight *wv,
                   const int8_t *quants, const float *scales, const int32_t *sums, float *q, float *k, float *v) {
    JL_REQUIRE(ctx && wq && wk && wv && quants && scales && sums && q && k && v, "jl_gemv_qkv_q8: null argument");
    if (wq->type != wk->type || wq->type != wv->type) {
        return jl_fail(JL_ERR_UNSUPPORTED, "jl_gemv_qkv_q8: no fused q|k|v kernel for mixed weights %s/%s/%s",
                       jl_type_name(wq->type), jl_type_name(wk->type), jl_type_name(wv->type));
    }
    JL_REQUIRE(wq->cols == wk->cols && wq->cols == wv->cols, "jl_gemv_qkv_q8: row lengths differ (%lld, %lld, %lld)",
               (long long)wq->cols, (long long)wk->cols, (long long)wv->cols);
    const jl_weight *ws[3] = {wq, wk, wv};
    float *outs[3] = {q, k, v};
    const jl_q8x xq{quants, scales, sums};
    return jl_launch_gemv(ctx, ws, 3, outs, nullptr, nullptr, JL_STORE, nullptr, &xq);
}

int jl_gemv_gate_up_q8(jl_context *ctx, const jl_weight *w1, const jl_weight *w3, const int8_t *quants,
                       const float *scales, const int32_t *sums, float *hb) {
    JL_REQUIRE(ctx && w1 && w3 && quants && scales && sums && hb, "jl_gemv_gate_up_q8: null argument");
    if (w1->type != w3->type) {
        return jl_fail(JL_ERR_UNSUPPORTED, "jl_gemv_gate_up_q8: no fused gate/up kernel for a %s gate and a %s up weight",
                       jl_type_name(w1->type), jl_type_name(w3->type));
    }
    JL_REQUIRE(w1->rows == w3->rows && w1->cols == w3->cols, "jl_gemv_gate_up_q8: gate is %lld x %lld, up is %lld x %lld",
               (long long)w1->rows, (long long)w1->cols, (long long)w3->rows, (long long)w3->cols);
    const jl_q8x xq{quants, scales, sums};
    return jl_launch_gemv(ctx, &w1, 1, &hb, w3, nullptr, JL_SWIGLU, nullptr, &xq);
}

int jl_argmax(jl_context *ctx, const float *values, int64_t n, int32_t *index) {
    JL_REQUIRE(ctx && values && index && n > 0 && n <= INT32_MAX, "jl_argmax: bad argument");
    return jl_launch_argmax(ctx, values, n, index);
}

int jl_gemv_argmax(jl_context *ctx, const jl_weight *w, const float *x, const float *rms_weights,
                   const float *rms_scale, float eps, float *out, int32_t *index) {
    JL_REQUIRE(ctx && w && x && out && index, "jl_gemv_argmax: null argument");
    JL_REQUIRE(w->rows <= INT32_MAX, "jl_gemv_argmax: %lld rows", (long long)w->rows);
    const jl_rms rms{rms_weights, rms_scale, eps};
    return jl_launch_gemv_argmax(ctx, w, x, rms_weights ? &rms : nullptr, out, index);
}

int jl_argmax_rows(jl_context *ctx, const float *values, int64_t rows, int64_t n, int64_t row_stride,
                   int32_t *indices) {
    JL_REQUIRE(ctx && values && indices, "jl_argmax_rows: null argument");
    JL_REQUIRE(rows >= 0 && rows <= INT32_MAX && n > 0 && n <= INT32_MAX && row_stride >= n,
               "jl_argmax_rows: %lld rows of %lld values, %lld apart", (long long)rows, (long long)n,
               (long long)row_stride);
    if (rows == 0) return JL_OK;
    return jl_launch_argmax_rows(ctx, values, rows, n, row_stride, indices);
}

int jl_argmax_static(jl_context *ctx, const float *values, int64_t n, int32_t *index) {
    JL_REQUIRE(ctx && values && index, "jl_argmax_static: null argument");
    JL_REQUIRE(n > 0, "jl_argmax_static: %lld values", (long long)n);
    JL_REQUIRE(n <= JL_ARGMAX_STATIC_MAX_VALUES, "jl_argmax_static: %lld values, at most %lld (use jl_argmax)",
               (long long)n, (long long)JL_ARGMAX_STATIC_MAX_VALUES);
    return jl_launch_argmax_static(ctx, values, n, index);
}

int jl_swiglu(jl_context *ctx, float *gate, const float *up, int64_t count) {
    JL_REQUIRE(ctx && gate && up && count >= 0, "jl_swiglu: bad argument");
    if (!count) return JL_OK;
    return jl_launch_swiglu(ctx, gate, up, count);
}

int jl_residual_add(jl_context *ctx, float *residual, const float *delta, int64_t count) {
    JL_REQUIRE(ctx && residual && delta && count >= 0 && count <= (int64_t)UINT32_MAX * 256,
               "jl_residual_add: bad argument");
    if (!count) return JL_OK;
    return jl_launch_residual_add(ctx, residual, delta, count);
}

size_t jl_gemm_workspace_bytes(int64_t max_rows, int64_t cols, int64_t out_cols, int math) {
    if (max_rows <= 0 || cols <= 0 || out_cols < 0) return 0;
    return jl_gemm_workspace_bytes_impl(max_rows, cols, out_cols, math == JL_MATH_DEFAULT ? JL_MATH_F16 : math);
}

static int gemm_checked(jl_context *ctx, const jl_weight *const *weights, int count, const float *X, float *C,
                        int64_t batch, int64_t active_rows, int64_t ldo, int64_t col_offset, int epilogue,
                        int math, void *workspace, size_t workspace_bytes, const jl_resident *resident,
                        const jl_half_io *half = nullptr) {
    JL_REQUIRE(ctx && weights && (X || (half && half->x16)) && C, "jl_gemm: null argument");
    JL_REQUIRE(!(half && half->c_f16) || epilogue == JL_SWIGLU,
               "jl_gemm_xf16: only the JL_SWIGLU result can be written as fp16 (epilogue %d)", epilogue);
    JL_REQUIRE(count >= 1 && count <= 8, "jl_gemm: %d weights (1..8)", count);
    JL_REQUIRE(batch >= 1 && active_rows >= 0 && active_rows <= batch,
               "jl_gemm: active_rows %lld of batch %lld", (long long)active_rows, (long long)batch);
    JL_REQUIRE(epilogue == JL_STORE || epilogue == JL_RESIDUAL || epilogue == JL_SWIGLU,
               "jl_gemm: epilogue %d", epilogue);
    int64_t total = 0;
    for (int i = 0; i < count; i++) {
        JL_REQUIRE(weights[i] != nullptr, "jl_gemm: weight %d is null", i);
        // (weights of different types run the decode-once path, each decoded by its own type; the
        // int8 mode multiplies the raw blocks and has no such path)
        if (weights[i]->type != weights[0]->type && math == JL_MATH_INT8) {
            return jl_fail(JL_ERR_UNSUPPORTED, "jl_gemm: mixed weight types %s and %s in one int8 call",
                           jl_type_name(weights[0]->type), jl_type_name(weights[i]->type));
        }
        JL_REQUIRE(weights[i]->cols == weights[0]->cols, "jl_gemm: weight %d row length %lld != %lld",
                   i, (long long)weights[i]->cols, (long long)weights[0]->cols);
        total += weights[i]->rows;
    }
    if (epilogue == JL_SWIGLU) {
        JL_REQUIRE(count == 2 && weights[0]->rows == weights[1]->rows,
                   "jl_gemm: JL_SWIGLU takes a gate and an up weight of equal shape");
        total = weights[0]->rows;
    }
    JL_REQUIRE(col_offset >= 0 && ldo >= col_offset + total,
               "jl_gemm: ldo %lld < col_offset %lld + %lld output columns", (long long)ldo,
               (long long)col_offset, (long long)total);
    if (math == JL_MATH_DEFAULT) math = JL_MATH_F16;
    JL_REQUIRE(math == JL_MATH_F16 || math == JL_MATH_INT8, "jl_gemm: math %d", math);
    if (math == JL_MATH_INT8 && weights[0]->type == JL_Q4_K) {
        return jl_fail(JL_ERR_UNSUPPORTED,
                       "jl_gemm: no int8 kernel for a Q4_K weight (d*sc*q - dmin*m is not an int8 "
                       "value); use JL_MATH_F16");
    }
    if (active_rows == 0) return JL_OK;
    // the activation copy and the row scales are mandatory; split-K planes are used if they fit
    size_t need = jl_gemm_workspace_bytes_impl(batch, weights[0]->cols, 0, math);
    if (workspace_bytes < need || (need && !workspace)) {
        return jl_fail(JL_ERR_WORKSPACE, "jl_gemm: workspace %zu bytes, %zu needed", workspace_bytes,
                       need);
    }
    return jl_launch_gemm(ctx, weights, count, X, C, batch, active_rows, ldo, col_offset, epilogue,
                          math, workspace, workspace_bytes, resident, half);
}

int jl_gemm(jl_context *ctx, const jl_weight *const *weights, int count, const float *X, float *C,
            int64_t batch, int64_t active_rows, int64_t ldo, int64_t col_offset, int epilogue,
            int math, void *workspace, size_t workspace_bytes) {
    return gemm_checked(ctx, weights, count, X, C, batch, active_rows, ldo, col_offset, epilogue, math,
                        workspace, workspace_bytes, nullptr);
}

size_t jl_gemm_resident_bytes(const jl_weight *const *weights, int count) {
    if (!weights || count < 1) return 0;
    int64_t rows = 0;
    for (int i = 0; i < count; i++) {
        if (!weights[i]) return 0;
        rows += weights[i]->rows;
    }
    // 2 bytes per weight, rows padded to whole 256-row tiles of either layout
    return (size_t)((rows + 511) / 256 * 256) * (size_t)weights[0]->cols * 2;
}

int jl_gemm_resident(jl_context *ctx, const jl_weight *const *weights, int count, const float *X, float *C,
                     int64_t batch, int64_t active_rows, int64_t ldo, int64_t col_offset, int epilogue,
                     int math, void *workspace, size_t workspace_bytes, void *resident,
                     size_t resident_bytes, int32_t *resident_state) {
    JL_REQUIRE(resident && resident_state, "jl_gemm_resident: null resident buffer or state");
    JL_REQUIRE(((uintptr_t)resident & 255) == 0, "jl_gemm_resident: the resident buffer must be 256-byte aligned");
    const jl_resident r{resident, resident_bytes, resident_state};
    return gemm_checked(ctx, weights, count, X, C, batch, active_rows, ldo, col_offset, epilogue, math,
                        workspace, workspace_bytes, &r);
}

int jl_rms_apply_xf16(jl_context *ctx, float *X, const float *delta, const float *rms_weights, float eps,
                      int64_t rows, int64_t n, float *scales, uint16_t *out) {
    JL_REQUIRE(ctx && X && rms_weights && out, "jl_rms_apply_xf16: null argument");
    JL_REQUIRE(rows >= 0 && n > 0 && n <= INT32_MAX && rows <= INT32_MAX, "jl_rms_apply_xf16: %lld rows of %lld",
               (long long)rows, (long long)n);
    if (rows == 0) return JL_OK;
    return jl_launch_rms_apply_f16(ctx, X, delta, rms_weights, eps, rows, n, scales, (_Float16 *)out);
}

int jl_gemm_xf16(jl_context *ctx, const jl_weight *const *weights, int count, const uint16_t *X, void *C,
                 int c_fp16, int64_t batch, int64_t active_rows, int64_t ldo, int64_t col_offset, int epilogue,
                 void *workspace, size_t workspace_bytes, void *resident, size_t resident_bytes,
                 int32_t *resident_state) {
    JL_REQUIRE(X != nullptr, "jl_gemm_xf16: null argument");
    JL_REQUIRE((resident == nullptr) == (resident_state == nullptr),
               "jl_gemm_xf16: a resident buffer and its state go together");
    JL_REQUIRE(((uintptr_t)resident & 255) == 0, "jl_gemm_xf16: the resident buffer must be 256-byte aligned");
    const jl_resident r{resident, resident_bytes, resident_state};
    const jl_half_io half{(const _Float16 *)X, c_fp16 != 0};
    return gemm_checked(ctx, weights, count, nullptr, (float *)C, batch, active_rows, ldo, col_offset, epilogue,
                        JL_MATH_F16, workspace, workspace_bytes, resident ? &r : nullptr, &half);
}

}  // extern "C"
