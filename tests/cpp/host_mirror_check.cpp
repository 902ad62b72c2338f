// The C++ host side (include/jitllm_hip.hpp) exercised as a C++ program: the reference's projection
// seams called by their own names, every result held to the CPU oracle on the same seeded inputs.
// Built by __graft_entry__.build() beside the library; run by tests/test_cpp_host.py.
//
//   host_mirror_check --no-device    argument checks and exception types only (no GPU needed)
//   host_mirror_check                the parity checks on device 0; prints one line per case
#include <unistd.h>

#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <string>
#include <vector>

#include "jitllm_hip.hpp"
#include "jitllm_oracle.h"

using namespace jitllm;

namespace {

// splitmix64: one seed, one tensor
struct Rng {
    std::uint64_t s;
    std::uint64_t next() {
        std::uint64_t z = (s += 0x9E3779B97F4A7C15ull);
        z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
        z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
        return z ^ (z >> 31);
    }
    double uniform() { return (double)(next() >> 11) * (1.0 / 9007199254740992.0); }
    float normal() {   // Box-Muller
        const double u = uniform() + 1e-300, v = uniform();
        return (float)(std::sqrt(-2.0 * std::log(u)) * std::cos(6.283185307179586 * v));
    }
};

// Blocks with fp16 scales in [1e-3, 2e-2] and uniformly random quants; the K-quant super-block's
// 6-bit scale bytes are random too (every bit pattern is a valid block).
std::vector<std::uint8_t> weight(int type, int rows, int cols, std::uint64_t seed) {
    Rng rng{seed};
    const int be = jo_block_elems(type), bb = jo_block_bytes(type);
    const std::int64_t blocks = (std::int64_t)rows * (cols / be);
    std::vector<std::uint8_t> raw((std::size_t)(blocks * bb));
    for (std::int64_t b = 0; b < blocks; b++) {
        std::uint8_t *p = raw.data() + b * bb;
        for (int i = 0; i < bb; i += 8) {
            const std::uint64_t r = rng.next();
            std::memcpy(p + i, &r, (std::size_t)(bb - i < 8 ? bb - i : 8));
        }
        const std::uint16_t d = jo_f32_to_f16((float)(1e-3 + rng.uniform() * 1.9e-2));
        std::memcpy(p + (type == JO_Q6_K ? 208 : 0), &d, 2);   // (a Q6_K super-block ends with its scale)
        if (type == JO_Q4_K) {
            const std::uint16_t dmin = jo_f32_to_f16((float)(1e-3 + rng.uniform() * 1.9e-2) / 16.f);
            std::memcpy(p + 2, &dmin, 2);
        }
    }
    return raw;
}

std::vector<float> activations(std::size_t n, std::uint64_t seed) {
    Rng rng{seed};
    std::vector<float> x(n);
    for (auto &v : x) v = rng.normal();
    return x;
}

// sum_j |w_ij x_j| per output, the scale errors are held against
std::vector<double> magnitude(int type, const std::vector<std::uint8_t> &raw, const float *x, int d, int n) {
    std::vector<float> w((std::size_t)d * n);
    jo_dequant(type, raw.data(), (std::int64_t)d * n, w.data());
    std::vector<double> m((std::size_t)d, 0.0);
    for (int i = 0; i < d; i++)
        for (int j = 0; j < n; j++) m[(std::size_t)i] += std::fabs((double)w[(std::size_t)i * n + j] * x[j]);
    return m;
}

int failures = 0;

void held(const char *name, const float *got, const float *want, const double *mag, std::size_t count, double bound) {
    double worst = 0.0;
    for (std::size_t i = 0; i < count; i++) {
        const double e = std::fabs((double)got[i] - (double)want[i]) / (mag[i] > 1e-30 ? mag[i] : 1e-30);
        if (!(e <= worst)) worst = e;   // (a NaN stays)
    }
    const bool ok = worst < bound;
    std::printf("[cpp-host] %-44s %s  (%.2e of the magnitude sum, bound %.0e)\n", name, ok ? "ok" : "FAILED", worst, bound);
    std::fflush(stdout);
    if (!ok) failures++;
}

void expect(const char *name, bool ok) {
    std::printf("[cpp-host] %-44s %s\n", name, ok ? "ok" : "FAILED");
    std::fflush(stdout);
    if (!ok) failures++;
}

// the dot the host runs for a type: the 256-bit vector one for Q8_0 and Q4_0, the scalar one otherwise
int flavour(int type) { return type == JO_Q8_0 || type == JO_Q4_0 ? JO_DOT_VEC256 : JO_DOT_SCALAR; }

int no_device() {
    // what needs no GPU: a context on a machine without one fails with a status and a message, and
    // the size query and the shape checks answer on the host
    bool threw = false;
    try {
        Context context(0);
    } catch (const Error &e) {
        threw = e.status() < 0 && std::strlen(e.what()) > 0;
    }
    expect("no device: Context throws jitllm::Error", threw);
    expect("no device: workspace query", jl_gemm_workspace_bytes(64, 4096, 4096, JL_MATH_DEFAULT) > 0);
    threw = false;
    try {
        check(jl_gemv(nullptr, nullptr, nullptr, nullptr, JL_STORE));
    } catch (const UnsupportedProjection &) {
    } catch (const Error &e) {
        threw = e.status() == JL_ERR_INVALID;
    }
    expect("no device: a null argument is JL_ERR_INVALID", threw);
    expect("no device: the split-K switch wants a context", jl_context_set_split_k(nullptr, 0) == JL_ERR_INVALID);
    return failures ? 1 : 0;
}

}  // namespace

int main(int argc, char **argv) {
    if (argc > 1 && std::string(argv[1]) == "--no-device") return no_device();
    const int threads = jo_max_threads();
    Context ctx(0);

    // ---- decode: one activation vector --------------------------------------------------------
    for (int type : {JO_Q8_0, JO_Q4_0, JO_Q4_K, JO_Q6_K}) {
        const int d = 264, n = 2048;
        const std::string tag = " type " + std::to_string(type);
        const auto raw = weight(type, d, n, 100 + (std::uint64_t)type);
        const auto x = activations((std::size_t)n, 200);
        const auto mag = magnitude(type, raw, x.data(), d, n);
        std::vector<float> ref((std::size_t)d);
        jo_matmul(type, flavour(type), raw.data(), x.data(), ref.data(), d, n, threads);
        TornadoTensor w(ctx, type, raw.data(), d, n);
        expect(("dequantize = getFloat, bit for bit," + tag).c_str(), [&] {
            const auto got = w.dequantize(ctx);
            std::vector<float> want(got.size());
            jo_dequant(type, raw.data(), (std::int64_t)got.size(), want.data());
            return std::memcmp(got.data(), want.data(), got.size() * sizeof(float)) == 0;
        }());
        const auto base = activations((std::size_t)d, 201);
        FloatArray dx(ctx, x), out(ctx, (std::size_t)d), acc(ctx, base);
        TornadoWorkspace ws;
        ws.wrapX = &acc;
        ws.wrapXb = &dx;
        QuantizedProjections proj(ctx, ws);
        proj.matvec(out, w, n, d);
        proj.residualMatvec(dx, w, n, d);
        ctx.sync();
        held(("matvec," + tag).c_str(), out.get().data(), ref.data(), mag.data(), (std::size_t)d, 2e-5);
        std::vector<float> sum((std::size_t)d);
        for (int i = 0; i < d; i++) sum[(std::size_t)i] = ref[(std::size_t)i] + base[(std::size_t)i];
        held(("residualMatvec," + tag).c_str(), acc.get().data(), sum.data(), mag.data(), (std::size_t)d, 2e-5);
    }
    {
        // fused q|k|v, fused and unfused gate/up, the unfused and the folded normalisation, argmax
        const int type = JO_Q8_0, n = 2048, dq = 512, dkv = 128, dff = 768;
        const auto rq = weight(type, dq, n, 301), rk = weight(type, dkv, n, 302), rv = weight(type, dkv, n, 303);
        const auto r1 = weight(type, dff, n, 304), r3 = weight(type, dff, n, 305), r3b = weight(JO_Q4_0, dff, n, 306);
        const auto x = activations((std::size_t)n, 310);
        auto rmsw = activations((std::size_t)n, 311);
        for (auto &v : rmsw) v = 1.f + 0.1f * v;
        TornadoTensor wq(ctx, type, rq.data(), dq, n), wk(ctx, type, rk.data(), dkv, n), wv(ctx, type, rv.data(), dkv, n);
        TornadoTensor w1(ctx, type, r1.data(), dff, n), w3(ctx, type, r3.data(), dff, n), w3b(ctx, JO_Q4_0, r3b.data(), dff, n);
        FloatArray dx(ctx, x), dxb(ctx, (std::size_t)n), q(ctx, (std::size_t)dq), k(ctx, (std::size_t)dkv), v(ctx, (std::size_t)dkv);
        FloatArray hb(ctx, (std::size_t)dff), hb2(ctx, (std::size_t)dff), drw(ctx, rmsw), scale(ctx, 1);
        DeviceBuffer token(ctx, 4);
        TornadoWorkspace ws;
        ws.wrapX = &dx;
        ws.wrapXb = &dx;     // the projections read x itself ...
        ws.wrapHb = &hb;
        ws.wrapHb2 = &hb2;
        QuantizedProjections proj(ctx, ws);
        proj.fusedQKV(dx, q, k, v, wq, wk, wv);
        ctx.sync();
        std::vector<float> ref((std::size_t)dq);
        jo_matmul(type, flavour(type), rq.data(), x.data(), ref.data(), dq, n, threads);
        held("fusedQKV: q", q.get().data(), ref.data(), magnitude(type, rq, x.data(), dq, n).data(), (std::size_t)dq, 2e-5);
        ref.resize((std::size_t)dkv);
        jo_matmul(type, flavour(type), rv.data(), x.data(), ref.data(), dkv, n, threads);
        held("fusedQKV: v", v.get().data(), ref.data(), magnitude(type, rv, x.data(), dkv, n).data(), (std::size_t)dkv, 2e-5);

        std::vector<float> g((std::size_t)dff), u((std::size_t)dff);
        auto swiglu_check = [&](const char *name, int up_type, const std::vector<std::uint8_t> &up_raw) {
            jo_matmul(type, flavour(type), r1.data(), x.data(), g.data(), dff, n, threads);
            jo_matmul(up_type, flavour(up_type), up_raw.data(), x.data(), u.data(), dff, n, threads);
            const auto mg = magnitude(type, r1, x.data(), dff, n), mu = magnitude(up_type, up_raw, x.data(), dff, n);
            std::vector<double> bound((std::size_t)dff);
            for (int i = 0; i < dff; i++)
                bound[(std::size_t)i] = mg[(std::size_t)i] * std::fabs(u[(std::size_t)i]) + 1.2 * mu[(std::size_t)i] * std::fabs(g[(std::size_t)i]) + 1e-6;
            std::vector<float> want = g;
            jo_swiglu(want.data(), u.data(), dff);
            held(name, hb.get().data(), want.data(), bound.data(), (std::size_t)dff, 2e-5);
        };
        expect("fusedGateUp: a Q8_0 pair is fused, Q8_0 + Q4_0 not", proj.fusedGateUp(w1, w3) && !proj.fusedGateUp(w1, w3b));
        proj.gateUp(w1, w3, n, dff);
        ctx.sync();
        swiglu_check("gateUp, one launch", type, r3);
        proj.gateUp(w1, w3b, n, dff);
        ctx.sync();
        swiglu_check("gateUp, two projections and SwiGLU", JO_Q4_0, r3b);

        // rmsScale + rmsApply + matvec against rmsnorm + matVec; the folded form against the same
        std::vector<float> xn((std::size_t)n);
        jo_rmsnorm(xn.data(), x.data(), rmsw.data(), n, 1e-5f);
        ws.wrapXb = &dxb;
        QuantizedProjections normed(ctx, ws);
        normed.rmsScale(dx, n, 1e-5f, scale);
        normed.rmsApply(drw, scale, n);
        normed.matvec(q, wq, n, dq);
        ctx.sync();
        ref.resize((std::size_t)dq);
        jo_matmul(type, flavour(type), rq.data(), xn.data(), ref.data(), dq, n, threads);
        const auto magn = magnitude(type, rq, xn.data(), dq, n);
        held("rmsScale, rmsApply, matvec", q.get().data(), ref.data(), magn.data(), (std::size_t)dq, 2e-5);
        q.init(-1.f);
        normed.rmsMatvec(dx, drw, nullptr, q, wq, n, dq, 1e-5f);
        ctx.sync();
        held("rmsMatvec (scale in the kernel)", q.get().data(), ref.data(), magn.data(), (std::size_t)dq, 2e-5);
        normed.matvecArgmax(dx, q, wq, n, dq, token, &drw, nullptr, 1e-5f);
        ctx.sync();
        std::int32_t tok = -1;
        token.download(&tok, 4);
        const auto logits = q.get();
        expect("matvecArgmax: the first maximum of its logits", tok == (std::int32_t)jo_argmax(logits.data(), dq));

        bool refused = false;
        try {
            proj.fusedQKV(dx, hb, hb, hb, w1, w1, w3b);   // Q8_0, Q8_0, Q4_0 in one single-token launch
        } catch (const UnsupportedProjection &e) {
            refused = std::strstr(e.what(), "mixed") != nullptr;
        }
        expect("fusedQKV of mixed types throws UnsupportedProjection", refused);
    }

    // ---- batched rows -------------------------------------------------------------------------
    for (int B : {8, 40, 200}) {
        // (the largest batch with every GEMM kept whole, as under -Djitllm.prefill.splitK=false)
        ctx.setSplitK(B != 200);
        const int n = 1024, dq = 520, dkv = 136, dff = 600;
        const std::string tag = " B " + std::to_string(B);
        const auto rq = weight(JO_Q4_K, dq, n, 401), rk = weight(JO_Q4_K, dkv, n, 402), rv = weight(JO_Q6_K, dkv, n, 403);
        const auto r1 = weight(JO_Q8_0, dff, n, 404), r3 = weight(JO_Q8_0, dff, n, 405);
        TornadoTensor wq(ctx, JO_Q4_K, rq.data(), dq, n), wk(ctx, JO_Q4_K, rk.data(), dkv, n), wv(ctx, JO_Q6_K, rv.data(), dkv, n);
        TornadoTensor w1(ctx, JO_Q8_0, r1.data(), dff, n), w3(ctx, JO_Q8_0, r3.data(), dff, n);
        const auto X = activations((std::size_t)B * n, 410 + (std::uint64_t)B);
        const int active = B - B / 5;
        FloatArray dX(ctx, X), qkv(ctx, (std::size_t)B * (dq + 2 * dkv)), hb(ctx, (std::size_t)B * dff);
        qkv.init(-12345.5f);
        hb.init(-12345.5f);
        QuantizedBatchProjections batch(ctx, B, n, 2 * dff);
        batch.fusedQKV(dX, qkv, wq, wk, wv, active);        // v of another type than q and k: one call
        batch.gateUp(dX, hb, w1, w3, n, dff, active);
        ctx.sync();
        const auto got = qkv.get();
        const int ld = dq + 2 * dkv;
        bool untouched = true;
        for (int b = active; b < B; b++)
            for (int j = 0; j < ld; j++) untouched = untouched && got[(std::size_t)b * ld + j] == -12345.5f;
        expect(("rows past activeRows are left alone," + tag).c_str(), untouched);
        struct Part { int type; const std::vector<std::uint8_t> *raw; int d, col; };
        for (const Part &p : {Part{JO_Q4_K, &rq, dq, 0}, Part{JO_Q4_K, &rk, dkv, dq}, Part{JO_Q6_K, &rv, dkv, dq + dkv}}) {
            std::vector<float> ref((std::size_t)active * p.d), mine((std::size_t)active * p.d);
            jo_matmul_batch(p.type, flavour(p.type), p.raw->data(), X.data(), ref.data(), active, p.d, n, threads);
            std::vector<double> mag;
            for (int b = 0; b < active; b++) {
                const auto m = magnitude(p.type, *p.raw, X.data() + (std::size_t)b * n, p.d, n);
                mag.insert(mag.end(), m.begin(), m.end());
                for (int j = 0; j < p.d; j++) mine[(std::size_t)b * p.d + j] = got[(std::size_t)b * ld + p.col + j];
            }
            held(("batched fusedQKV, column " + std::to_string(p.col) + "," + tag).c_str(), mine.data(), ref.data(), mag.data(),
                 mine.size(), 2e-3);
        }
        std::vector<float> g((std::size_t)active * dff), u((std::size_t)active * dff);
        jo_matmul_batch(JO_Q8_0, JO_DOT_VEC256, r1.data(), X.data(), g.data(), active, dff, n, threads);
        jo_matmul_batch(JO_Q8_0, JO_DOT_VEC256, r3.data(), X.data(), u.data(), active, dff, n, threads);
        std::vector<double> bound;
        for (int b = 0; b < active; b++) {
            const auto mg = magnitude(JO_Q8_0, r1, X.data() + (std::size_t)b * n, dff, n);
            const auto mu = magnitude(JO_Q8_0, r3, X.data() + (std::size_t)b * n, dff, n);
            for (int j = 0; j < dff; j++) {
                const std::size_t at = (std::size_t)b * dff + j;
                bound.push_back(mg[(std::size_t)j] * std::fabs(u[at]) + 1.2 * mu[(std::size_t)j] * std::fabs(g[at]) + 1e-6);
            }
        }
        std::vector<float> want = g;
        jo_swiglu(want.data(), u.data(), (std::int64_t)want.size());
        held(("batched gateUp," + tag).c_str(), hb.get().data(), want.data(), bound.data(), want.size(), 2e-3);

        // the prefill plan's operand types: RMS norm into fp16 rows, then the projection over them
        auto rmsw = activations((std::size_t)n, 420);
        for (auto &v : rmsw) v = 1.f + 0.1f * v;
        FloatArray drw(ctx, rmsw), scales(ctx, (std::size_t)B), out(ctx, (std::size_t)B * dq);
        HalfFloatArray xb16(ctx, (std::size_t)B * n);
        batch.rmsApplyFP16(dX, drw, 1e-5f, xb16, n, &scales);
        batch.projection(xb16, out, wq, n, dq, false);
        ctx.sync();
        std::vector<float> xcopy = X, sc((std::size_t)B);
        std::vector<std::uint16_t> want16((std::size_t)B * n);
        jo_batched_rms_apply_f16(xcopy.data(), nullptr, rmsw.data(), 1e-5f, B, n, sc.data(), want16.data());
        const auto got16 = xb16.get();
        expect(("rmsApplyFP16: the oracle's fp16 rows, bit for bit," + tag).c_str(),
               std::memcmp(got16.data(), want16.data(), got16.size() * 2) == 0);
        std::vector<float> x32(got16.size());
        for (std::size_t i = 0; i < x32.size(); i++) x32[i] = jo_f16_to_f32(got16[i]);
        std::vector<float> ref((std::size_t)B * dq);
        jo_matmul_batch(JO_Q4_K, JO_DOT_SCALAR, rq.data(), x32.data(), ref.data(), B, dq, n, threads);
        std::vector<double> mag;
        for (int b = 0; b < B; b++) {
            const auto m = magnitude(JO_Q4_K, rq, x32.data() + (std::size_t)b * n, dq, n);
            mag.insert(mag.end(), m.begin(), m.end());
        }
        held(("projection over fp16 rows," + tag).c_str(), out.get().data(), ref.data(), mag.data(), ref.size(), 2e-3);
        // one token per row of those outputs, as the batched logits graph ends
        DeviceBuffer tokens(ctx, (std::size_t)B * 4);
        batch.argmaxLogits(out, dq, tokens);
        ctx.sync();
        std::vector<std::int32_t> tok((std::size_t)B);
        tokens.download(tok.data(), tok.size() * 4);
        const auto rows = out.get();
        bool first_maxima = true;
        for (int b = 0; b < B; b++) first_maxima = first_maxima && tok[(std::size_t)b] == (std::int32_t)jo_argmax(rows.data() + (std::size_t)b * dq, dq);
        expect(("argmaxLogits: every row's first maximum," + tag).c_str(), first_maxima);
    }
    {
        // ---- a weight straight from a GGUF file ----------------------------------------------
        // version 3, one key (general.alignment = 32, u32), one Q8_0 tensor of ne = [256, 24]
        const int d = 24, n = 256;
        const auto raw = weight(JO_Q8_0, d, n, 501);
        std::string blob;
        auto put = [&](const void *p, std::size_t bytes) { blob.append(static_cast<const char *>(p), bytes); };
        auto put_u32 = [&](std::uint32_t v) { put(&v, 4); };
        auto put_u64 = [&](std::uint64_t v) { put(&v, 8); };
        auto put_str = [&](const std::string &t) { put_u64(t.size()); put(t.data(), t.size()); };
        put("GGUF", 4); put_u32(3); put_u64(1); put_u64(1);
        put_str("general.alignment"); put_u32(4 /* u32 */); put_u32(32);
        put_str("blk.0.attn_q.weight"); put_u32(2); put_u64((std::uint64_t)n); put_u64((std::uint64_t)d); put_u32(JO_Q8_0); put_u64(0);
        blob.append((32 - blob.size() % 32) % 32, '\0');
        put(raw.data(), raw.size());
        char path[] = "/tmp/jitllm_cpp_host_XXXXXX";
        const int fd = mkstemp(path);
        bool written = fd >= 0 && write(fd, blob.data(), blob.size()) == (ssize_t)blob.size();
        if (fd >= 0) close(fd);
        expect("a GGUF file written", written);
        if (written) {
            GGUF file(path);
            expect("GGUF: one tensor, found by name, alignment read",
                   file.tensorCount() == 1 && file.has("blk.0.attn_q.weight") && !file.has("nope") &&
                       file.metadataInt("general.alignment") == 32);
            TornadoTensor w = file.load(ctx, "blk.0.attn_q.weight");
            expect("GGUF: the tensor's type and ne order", w.dataType() == JO_Q8_0 && w.rows() == d && w.cols() == n);
            const auto x = activations((std::size_t)n, 502);
            FloatArray dx(ctx, x), out(ctx, (std::size_t)d);
            QuantizedProjections(ctx, TornadoWorkspace{}).floatMatvec(dx, out, w, n, d);
            ctx.sync();
            std::vector<float> ref((std::size_t)d);
            jo_matmul(JO_Q8_0, JO_DOT_VEC256, raw.data(), x.data(), ref.data(), d, n, threads);
            held("floatMatvec over a weight loaded from GGUF", out.get().data(), ref.data(),
                 magnitude(JO_Q8_0, raw, x.data(), d, n).data(), (std::size_t)d, 2e-5);
            bool missing = false;
            try {
                file.load(ctx, "blk.9.nope");
            } catch (const Error &e) {
                missing = std::strstr(e.what(), "no tensor") != nullptr;
            }
            expect("GGUF: a missing tensor is named", missing);
            std::remove(path);
        }
    }
    std::printf("[cpp-host] %s\n", failures ? "FAILED" : "all ok");
    return failures ? 1 : 0;
}
