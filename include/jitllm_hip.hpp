// C++17 host side above the C ABI of jitllm_hip.h: the reference's projection seams with their own
// method names and argument meaning, for a host written in a compiled language.  Header-only; a
// program includes it and links libjitllm_hip.so.
//
//   QuantizedProjections       J/backend/tornado/layers/QuantizedProjections.java (decode: one
//                              activation vector; n = row length, d = output rows)
//   QuantizedBatchProjections  J/backend/tornado/layers/QuantizedBatchProjections.java (batchSize
//                              activation rows; batched decode and batched prefill)
//   TornadoTensor, FloatArray, HalfFloatArray, TornadoWorkspace
//                              the operand types of those classes (J/backend/tornado/tensor/
//                              TornadoTensor.java:17-101; TornadoVM's FloatArray / HalfFloatArray;
//                              J/backend/tornado/workspace/TornadoWorkspace.java)
//   GGUF                       J/format/GGUF.java:40-255, as far as a tensor's upload needs it
//
// Where the reference adds a task to a TaskGraph these enqueue a kernel on the context's stream, so
// the `graph` / `name` arguments of the reference disappear.  Error behaviour is the reference's: a
// combination with no kernel throws (UnsupportedProjection, the reference's IllegalStateException
// "no ... kernel for a ... weight"), nothing else is ever run in its place.
#pragma once

#include <cstddef>
#include <cstdint>
#include <stdexcept>
#include <string>
#include <utility>
#include <vector>

#include "jitllm_hip.h"

namespace jitllm {

// A negative jl_status with the library's message for it.
class Error : public std::runtime_error {
public:
    Error(int status, const std::string &message)
        : std::runtime_error("[jl_status " + std::to_string(status) + "] " + message), status_(status) {}
    int status() const { return status_; }

private:
    int status_;
};
// JL_ERR_UNSUPPORTED: the reference's "no ... kernel for a ... weight" IllegalStateException.
class UnsupportedProjection : public Error {
public:
    using Error::Error;
};

inline void check(int status) {
    if (status >= 0) return;
    const char *text = jl_last_error();
    const std::string message = text ? text : "";
    if (status == JL_ERR_UNSUPPORTED) throw UnsupportedProjection(status, message);
    throw Error(status, message);
}

// One device, one stream (the reference's execution plan owns one of each per program).
class Context {
public:
    explicit Context(int device = 0) { check(jl_context_create(device, &handle_)); }
    // on a stream the caller owns (a hipStream_t); the stream is borrowed
    Context(int device, void *hip_stream) { check(jl_context_create_on_stream(device, hip_stream, &handle_)); }
    ~Context() { jl_context_destroy(handle_); }
    Context(const Context &) = delete;
    Context &operator=(const Context &) = delete;
    jl_context *handle() const { return handle_; }
    void *stream() const { return jl_context_stream(handle_); }
    void sync() const { check(jl_sync(handle_)); }
    // false: every GEMM whole (-Djitllm.prefill.splitK=false, SplitKGemm.java:40-42)
    void setSplitK(bool enabled) const { check(jl_context_set_split_k(handle_, enabled ? 1 : 0)); }

private:
    jl_context *handle_ = nullptr;
};

// Untyped device memory (jl_malloc / jl_free).
class DeviceBuffer {
public:
    DeviceBuffer(const Context &context, std::size_t bytes) : context_(&context), bytes_(bytes) {
        check(jl_malloc(context.handle(), bytes, &ptr_));
    }
    ~DeviceBuffer() {
        if (ptr_) jl_free(context_->handle(), ptr_);
    }
    DeviceBuffer(const DeviceBuffer &) = delete;
    DeviceBuffer &operator=(const DeviceBuffer &) = delete;
    DeviceBuffer(DeviceBuffer &&other) noexcept : context_(other.context_), ptr_(other.ptr_), bytes_(other.bytes_) {
        other.ptr_ = nullptr;
    }
    void *ptr() const { return ptr_; }
    std::size_t bytes() const { return bytes_; }
    void upload(const void *host, std::size_t bytes, std::size_t offset = 0) const {
        if (offset + bytes > bytes_) throw std::out_of_range("upload past the end of the device buffer");
        check(jl_upload(context_->handle(), static_cast<char *>(ptr_) + offset, host, bytes));
    }
    void download(void *host, std::size_t bytes, std::size_t offset = 0) const {
        if (offset + bytes > bytes_) throw std::out_of_range("download past the end of the device buffer");
        check(jl_download(context_->handle(), host, static_cast<const char *>(ptr_) + offset, bytes));
    }

protected:
    const Context *context_;
    void *ptr_ = nullptr;
    std::size_t bytes_;
};

// fp32 device array; init / set / get as on TornadoVM's FloatArray.
class FloatArray : public DeviceBuffer {
public:
    FloatArray(const Context &context, std::size_t size) : DeviceBuffer(context, size * sizeof(float)), size_(size) {}
    FloatArray(const Context &context, const std::vector<float> &values) : FloatArray(context, values.size()) { set(values); }
    std::size_t size() const { return size_; }
    float *data() const { return static_cast<float *>(ptr_); }
    void init(float value) const { check(jl_fill_f32(context_->handle(), data(), value, size_)); }
    void set(const std::vector<float> &values) const {
        if (values.size() != size_) throw std::invalid_argument("values for a FloatArray of another size");
        upload(values.data(), size_ * sizeof(float));
    }
    std::vector<float> get() const {
        std::vector<float> out(size_);
        download(out.data(), size_ * sizeof(float));
        return out;
    }

private:
    std::size_t size_;
};

// binary16 device array (TornadoVM's HalfFloatArray): the operand type of the reference's prefill GEMMs.
class HalfFloatArray : public DeviceBuffer {
public:
    HalfFloatArray(const Context &context, std::size_t size) : DeviceBuffer(context, size * 2), size_(size) {}
    std::size_t size() const { return size_; }
    std::uint16_t *data() const { return static_cast<std::uint16_t *>(ptr_); }
    void set(const std::vector<std::uint16_t> &bits) const {
        if (bits.size() != size_) throw std::invalid_argument("values for a HalfFloatArray of another size");
        upload(bits.data(), size_ * 2);
    }
    std::vector<std::uint16_t> get() const {
        std::vector<std::uint16_t> out(size_);
        download(out.data(), size_ * 2);
        return out;
    }

private:
    std::size_t size_;
};

// A weight as the GGUF file stores it, resident on the device (TornadoTensor.java:17-101): uploaded
// once, consumed by handle afterwards.  `blocks` points at the first block, past any array header.
class TornadoTensor {
public:
    TornadoTensor(const Context &context, int ggml_type, const void *blocks, std::int64_t rows, std::int64_t cols) {
        check(jl_weight_upload(context.handle(), ggml_type, blocks, rows, cols, &handle_));
        check(jl_weight_info(handle_, &type_, &rows_, &cols_, &bytes_));
    }
    explicit TornadoTensor(jl_weight *adopted) : handle_(adopted) {
        check(jl_weight_info(handle_, &type_, &rows_, &cols_, &bytes_));
    }
    ~TornadoTensor() { jl_weight_free(handle_); }
    TornadoTensor(const TornadoTensor &) = delete;
    TornadoTensor &operator=(const TornadoTensor &) = delete;
    TornadoTensor(TornadoTensor &&other) noexcept
        : handle_(other.handle_), type_(other.type_), rows_(other.rows_), cols_(other.cols_), bytes_(other.bytes_) {
        other.handle_ = nullptr;
    }
    jl_weight *handle() const { return handle_; }
    int dataType() const { return type_; }
    std::int64_t rows() const { return rows_; }
    std::int64_t cols() const { return cols_; }
    std::int64_t bytes() const { return bytes_; }
    // the host tensor's getFloat over the whole weight, computed on the device (parity probe)
    std::vector<float> dequantize(const Context &context) const {
        FloatArray out(context, static_cast<std::size_t>(rows_ * cols_));
        check(jl_dequant_f32(context.handle(), handle_, out.data()));
        context.sync();
        return out.get();
    }

private:
    jl_weight *handle_ = nullptr;
    int type_ = 0;
    std::int64_t rows_ = 0, cols_ = 0, bytes_ = 0;
};

// A GGUF file's tensor table, and a tensor's upload straight from the mapped file.
class GGUF {
public:
    explicit GGUF(const std::string &path) { check(jl_gguf_open(path.c_str(), &handle_)); }
    ~GGUF() { jl_gguf_close(handle_); }
    GGUF(const GGUF &) = delete;
    GGUF &operator=(const GGUF &) = delete;
    std::int64_t tensorCount() const { return jl_gguf_tensor_count(handle_); }
    bool has(const std::string &name) const { return jl_gguf_find(handle_, name.c_str()) >= 0; }
    std::int64_t metadataInt(const std::string &key) const {
        std::int64_t value = 0;
        check(jl_gguf_metadata_int(handle_, key.c_str(), &value));
        return value;
    }
    TornadoTensor load(const Context &context, const std::string &name) const {
        jl_weight *w = nullptr;
        check(jl_gguf_upload(context.handle(), handle_, name.c_str(), &w));
        return TornadoTensor(w);
    }

private:
    jl_gguf *handle_ = nullptr;
};

// The persistent activation arrays a layer's projections read and write (TornadoWorkspace.java):
// bound once, values move, arrays never.
struct TornadoWorkspace {
    FloatArray *wrapX = nullptr;
    FloatArray *wrapXb = nullptr;
    FloatArray *wrapHb = nullptr;
    FloatArray *wrapHb2 = nullptr;
};

namespace detail {
inline void check_shape(const TornadoTensor &w, std::int64_t n, std::int64_t d) {
    if (w.cols() != n || w.rows() != d)
        throw std::invalid_argument("weight is " + std::to_string(w.rows()) + "x" + std::to_string(w.cols()) +
                                    ", projection asked for d=" + std::to_string(d) + ", n=" + std::to_string(n));
}
inline FloatArray &bound(FloatArray *array, const char *name) {
    if (!array) throw std::logic_error(std::string("the workspace has no ") + name + " bound");
    return *array;
}
}  // namespace detail

// Single-token projections over weights kept in the file's representations.
class QuantizedProjections {
public:
    QuantizedProjections(const Context &context, TornadoWorkspace workspace) : ctx_(context.handle()), ws_(workspace) {}

    // out = w . wrapXb (QuantizedProjections.java:140-194)
    void matvec(const FloatArray &out, const TornadoTensor &w, int n, int d) const {
        floatMatvec(detail::bound(ws_.wrapXb, "wrapXb"), out, w, n, d);
    }
    // out = w . x (:200-254)
    void floatMatvec(const FloatArray &x, const FloatArray &out, const TornadoTensor &w, int n, int d) const {
        detail::check_shape(w, n, d);
        check(jl_gemv(ctx_, w.handle(), x.data(), out.data(), JL_STORE));
    }
    // wrapX += w . x (:260-379)
    void residualMatvec(const FloatArray &x, const TornadoTensor &w, int n, int d) const {
        detail::check_shape(w, n, d);
        check(jl_gemv(ctx_, w.handle(), x.data(), detail::bound(ws_.wrapX, "wrapX").data(), JL_RESIDUAL));
    }
    // q | k | v in one launch (fusedQKVMatmulQ8 and its Q4_0 / Q4_K siblings, called directly on the
    // kernels by the reference's layer builders, LlamaQ8_0FFNLayers.java:316-329)
    void fusedQKV(const FloatArray &x, const FloatArray &q, const FloatArray &k, const FloatArray &v, const TornadoTensor &wq,
                  const TornadoTensor &wk, const TornadoTensor &wv) const {
        check(jl_gemv_qkv(ctx_, wq.handle(), wk.handle(), wv.handle(), x.data(), q.data(), k.data(), v.data()));
    }
    // QuantizedProjections.java:386-393: both weights of one type, Q8_0 / Q4_0 / Q4_K / Q5_K
    bool fusedGateUp(const TornadoTensor &w1, const TornadoTensor &w3) const {
        const int t = w1.dataType();
        return t == w3.dataType() && (t == JL_Q8_0 || t == JL_Q4_0 || t == JL_Q4_K || t == JL_Q5_K);
    }
    // wrapHb = SiLU(w1 . wrapXb) * (w3 . wrapXb) (:400-480): one fused launch where fusedGateUp
    // holds, else two projections into wrapHb and wrapHb2 and an element-wise SwiGLU
    void gateUp(const TornadoTensor &w1, const TornadoTensor &w3, int n, int d) const {
        detail::check_shape(w1, n, d);
        detail::check_shape(w3, n, d);
        const FloatArray &xb = detail::bound(ws_.wrapXb, "wrapXb"), &hb = detail::bound(ws_.wrapHb, "wrapHb");
        if (fusedGateUp(w1, w3)) {
            check(jl_gemv_gate_up(ctx_, w1.handle(), w3.handle(), xb.data(), hb.data()));
            return;
        }
        const FloatArray &hb2 = detail::bound(ws_.wrapHb2, "wrapHb2");
        matvec(hb, w1, n, d);
        matvec(hb2, w3, n, d);
        check(jl_swiglu(ctx_, hb.data(), hb2.data(), d));
    }

    // ---- the steps on either side of a projection ----

    // scale[0] = 1 / sqrt(sum x^2 / n + eps) on the device (reductionOneBlockWithLayer,
    // TransformerComputeKernels.java:378-437)
    void rmsScale(const FloatArray &x, int n, float eps, const FloatArray &scale) const {
        check(jl_rms_scale(ctx_, x.data(), n, eps, scale.data()));
    }
    // wrapXb = rmsWeights * (temp[0] * wrapX) (QuantizedProjections.rmsApply :117-130,
    // reductionOneBlock2WithLayer)
    void rmsApply(const FloatArray &rmsWeights, const FloatArray &temp, int n) const {
        check(jl_rms_apply(ctx_, detail::bound(ws_.wrapX, "wrapX").data(), rmsWeights.data(), temp.data(), n,
                           detail::bound(ws_.wrapXb, "wrapXb").data()));
    }
    // out = w . (rmsWeights * (s * x)), the final norm folded into the vocabulary projection
    // (reductionOneBlock2WithLogits + the projection, LogitsQ8_0Layer.java:85-97); s = rmsScale[0],
    // or with rmsScale null computed in the kernel from eps
    void rmsMatvec(const FloatArray &x, const FloatArray &rmsWeights, const FloatArray *rmsScale, const FloatArray &out,
                   const TornadoTensor &w, int n, int d, float eps = 0.f) const {
        detail::check_shape(w, n, d);
        check(jl_gemv_rms(ctx_, w.handle(), x.data(), rmsWeights.data(), rmsScale ? rmsScale->data() : nullptr, eps,
                          out.data(), JL_STORE));
    }
    // fusedRmsNormQKVMatmulQ8 (TransformerComputeKernelsLayered.java:2116-2220)
    void fusedRmsNormQKV(const FloatArray &x, const FloatArray &q, const FloatArray &k, const FloatArray &v,
                         const FloatArray &rmsWeights, const FloatArray *rmsScale, const TornadoTensor &wq,
                         const TornadoTensor &wk, const TornadoTensor &wv, float eps = 0.f) const {
        check(jl_gemv_qkv_rms(ctx_, wq.handle(), wk.handle(), wv.handle(), x.data(), rmsWeights.data(),
                              rmsScale ? rmsScale->data() : nullptr, eps, q.data(), k.data(), v.data()));
    }
    // fullyFusedRmsNormFFNGateUpQ8 (:2866+): wrapHb = SiLU(w1 . xn) * (w3 . xn), the scale computed in the kernel
    void fullyFusedRmsNormGateUp(const FloatArray &x, const FloatArray &rmsWeights, float eps, const TornadoTensor &w1,
                                 const TornadoTensor &w3, int n, int d) const {
        detail::check_shape(w1, n, d);
        detail::check_shape(w3, n, d);
        check(jl_gemv_gate_up_rms(ctx_, w1.handle(), w3.handle(), x.data(), rmsWeights.data(), eps,
                                  detail::bound(ws_.wrapHb, "wrapHb").data()));
    }
    // token[0] = index of the first maximum of the logits, an int32 on the device (argmaxLogits,
    // TransformerComputeKernels.java:95-127)
    void argmax(const FloatArray &logits, std::int64_t n, const DeviceBuffer &token) const {
        check(jl_argmax(ctx_, logits.data(), n, static_cast<std::int32_t *>(token.ptr())));
    }
    // the vocabulary projection followed by "argmax_sample" in one call (LogitsQ8_0Layer.java:92-110);
    // rmsWeights null for an already normalised x
    void matvecArgmax(const FloatArray &x, const FloatArray &logits, const TornadoTensor &w, int n, int d,
                      const DeviceBuffer &token, const FloatArray *rmsWeights = nullptr, const FloatArray *rmsScale = nullptr,
                      float eps = 0.f) const {
        detail::check_shape(w, n, d);
        check(jl_gemv_argmax(ctx_, w.handle(), x.data(), rmsWeights ? rmsWeights->data() : nullptr,
                             rmsScale ? rmsScale->data() : nullptr, eps, logits.data(),
                             static_cast<std::int32_t *>(token.ptr())));
    }

private:
    jl_context *ctx_;
    TornadoWorkspace ws_;
};

// Projections of batchSize activation rows at once (batched decode, batched prefill).
class QuantizedBatchProjections {
public:
    // maxCols: the longest row any projection reads; maxOutCols: the most output columns one call
    // produces (gate + up rows for a fused gate/up).  Together they size the workspace once, before
    // anything runs (Implementation.needs, J/backend/tornado/ops/Implementation.java:31-36).
    QuantizedBatchProjections(const Context &context, int batchSize, std::int64_t maxCols, std::int64_t maxOutCols,
                              int math = JL_MATH_DEFAULT)
        : ctx_(context.handle()), batch_(batchSize), math_(math),
          workspace_(context, workspace_bytes(batchSize, maxCols, maxOutCols, math)) {}

    int batchSize() const { return batch_; }
    std::size_t workspaceBytes() const { return workspace_.bytes(); }

    // tokens[b] = first maximum of row b of the batched logits, int32 on the device
    // (batchedArgmaxLogits, TransformerBatchPrefillKernels.java:2118-2159)
    void argmaxLogits(const FloatArray &logits, std::int64_t vocab, const DeviceBuffer &tokens, int activeRows = -1,
                      std::int64_t rowStride = -1) const {
        check(jl_argmax_rows(ctx_, logits.data(), activeRows < 0 ? batch_ : activeRows, vocab, rowStride < 0 ? vocab : rowStride,
                             static_cast<std::int32_t *>(tokens.ptr())));
    }
    // out = w . x over the batch, or out += w . x with `residual` (QuantizedBatchProjections.java:76-309);
    // rows past activeRows are left untouched
    void projection(const FloatArray &x, const FloatArray &out, const TornadoTensor &w, int n, int d, bool residual,
                    int activeRows = -1) const {
        detail::check_shape(w, n, d);
        const jl_weight *weights[1] = {w.handle()};
        gemm(weights, 1, x, out.data(), activeRows, d, residual ? JL_RESIDUAL : JL_STORE);
    }
    // out[b] = [wq . x_b | wk . x_b | wv . x_b], side by side (FP16Projections: C = A . [W0|W1|W2]^T);
    // the three weights may differ in type
    void fusedQKV(const FloatArray &x, const FloatArray &out, const TornadoTensor &wq, const TornadoTensor &wk,
                  const TornadoTensor &wv, int activeRows = -1) const {
        const jl_weight *weights[3] = {wq.handle(), wk.handle(), wv.handle()};
        gemm(weights, 3, x, out.data(), activeRows, wq.rows() + wk.rows() + wv.rows(), JL_STORE);
    }
    // QuantizedBatchProjections.java:315-321 (the tiled answer): one type, Q8_0 / Q4_0 / Q4_K
    bool fusedGateUp(const TornadoTensor &w1, const TornadoTensor &w3) const {
        const int t = w1.dataType();
        return t == w3.dataType() && (t == JL_Q8_0 || t == JL_Q4_0 || t == JL_Q4_K);
    }
    // hb = SiLU(w1 . x) * (w3 . x) over the batch (:329-458), one call for every pair of types; x is
    // already normalised
    void gateUp(const FloatArray &x, const FloatArray &hb, const TornadoTensor &w1, const TornadoTensor &w3, int dim,
                int hidDim, int activeRows = -1) const {
        detail::check_shape(w1, dim, hidDim);
        detail::check_shape(w3, dim, hidDim);
        const jl_weight *weights[2] = {w1.handle(), w3.handle()};
        gemm(weights, 2, x, hb.data(), activeRows, hidDim, JL_SWIGLU);
    }
    // out[b] = fp16(rmsWeights * scale_b * x[b]): batchedRmsReduceParallel + batchedRmsApplyFP16
    // (TransformerBatchPrefillKernels.java:1480-1510, 59-72), the producer of the prefill GEMMs'
    // fp16 activations; with `delta` the pending residual add x += delta comes first (:1519-1551)
    void rmsApplyFP16(const FloatArray &x, const FloatArray &rmsWeights, float eps, const HalfFloatArray &out, int dim,
                      const FloatArray *scales = nullptr, int activeRows = -1, const FloatArray *delta = nullptr) const {
        check(jl_rms_apply_xf16(ctx_, x.data(), delta ? delta->data() : nullptr, rmsWeights.data(), eps,
                                activeRows < 0 ? batch_ : activeRows, dim, scales ? scales->data() : nullptr, out.data()));
    }
    // the same calls over fp16 activations, the operand type of the reference's prefill plan
    // (DecodedMatMul.project, J/backend/tornado/ops/DecodedMatMul.java:100-109); `hidden16` set: the
    // gate/up + SwiGLU result as fp16 (batchedFFNSwiGLUFP16Packed)
    void projection(const HalfFloatArray &x, const FloatArray &out, const TornadoTensor &w, int n, int d, bool residual,
                    int activeRows = -1) const {
        detail::check_shape(w, n, d);
        const jl_weight *weights[1] = {w.handle()};
        gemm16(weights, 1, x, out.data(), false, activeRows, d, residual ? JL_RESIDUAL : JL_STORE);
    }
    void fusedQKV(const HalfFloatArray &x, const FloatArray &out, const TornadoTensor &wq, const TornadoTensor &wk,
                  const TornadoTensor &wv, int activeRows = -1) const {
        const jl_weight *weights[3] = {wq.handle(), wk.handle(), wv.handle()};
        gemm16(weights, 3, x, out.data(), false, activeRows, wq.rows() + wk.rows() + wv.rows(), JL_STORE);
    }
    void gateUp(const HalfFloatArray &x, const HalfFloatArray &hidden16, const TornadoTensor &w1, const TornadoTensor &w3,
                int dim, int hidDim, int activeRows = -1) const {
        detail::check_shape(w1, dim, hidDim);
        detail::check_shape(w3, dim, hidDim);
        const jl_weight *weights[2] = {w1.handle(), w3.handle()};
        gemm16(weights, 2, x, hidden16.data(), true, activeRows, hidDim, JL_SWIGLU);
    }

private:
    static std::size_t workspace_bytes(int batch, std::int64_t cols, std::int64_t out_cols, int math) {
        const std::size_t bytes = jl_gemm_workspace_bytes(batch, cols, out_cols, math);
        return bytes < 256 ? 256 : bytes;
    }
    void gemm(const jl_weight *const *weights, int count, const FloatArray &x, float *out, int activeRows, std::int64_t ldo,
              int epilogue) const {
        check(jl_gemm(ctx_, weights, count, x.data(), out, batch_, activeRows < 0 ? batch_ : activeRows, ldo, 0, epilogue,
                      math_, workspace_.ptr(), workspace_.bytes()));
    }
    void gemm16(const jl_weight *const *weights, int count, const HalfFloatArray &x, void *out, bool out16, int activeRows,
                std::int64_t ldo, int epilogue) const {
        check(jl_gemm_xf16(ctx_, weights, count, x.data(), out, out16 ? 1 : 0, batch_, activeRows < 0 ? batch_ : activeRows,
                           ldo, 0, epilogue, workspace_.ptr(), workspace_.bytes(), nullptr, 0, nullptr));
    }

    jl_context *ctx_;
    int batch_, math_;
    DeviceBuffer workspace_;
};

}  // namespace jitllm
