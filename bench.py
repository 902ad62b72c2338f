#!/usr/bin/env python3
"""Benchmark of the quantized weight-matmul hot path on one MI355X.

A step is one pass of the decode projection set of Llama-3.2-1B in Q8_0, batch 1 -- per layer the
fused q|k|v projection, the output projection (residual), the fused gate/up SwiGLU projection and
the down projection (residual), 16 layers, then the 2048 -> 128256 vocabulary projection: 65 kernel
launches, 1 316 320 256 algorithmic bytes (weights in GGUF block layout + fp32 input + fp32 output,
each once).  Inputs are resident in HBM before the timed region.  Every layer owns distinct device
buffers, so the 1.3 GB sweep cannot live in the 256 MB memory-side cache.

Prints one JSON line.  `value` is GB/s of algorithmic bytes; `roofline` is the largest single
launch shape of the step (the fused gate/up GEMV) against the 8 TB/s HBM peak; `cpu_baseline` is the
oracle's restatement of the reference's Java CPU matmul timed on this machine's host cores;
`prefill` and `batched` carry the MFMA side of the metric.

Every timed leg is a HIP graph replayed in REPS repetitions of K replays each; the figure reported
is the median repetition, its spread (max - min over the median) is given beside it and a spread
above 10 % is flagged "unstable" (the reference's rule, docs/architecture/verification.md:116-131).
Before a leg is timed, one of its outputs is downloaded and a sample of it compared with the CPU
oracle: a line cannot come from a kernel that computes something else.
"""
from __future__ import annotations

import argparse
import ctypes as C
import json
import os
import statistics
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0
F16_MFMA_PEAK_TFLOPS = 2500.0
INT8_MFMA_PEAK_TOPS = 5000.0
F16_MFMA_FLOPS_PER_CU_CLK = 4096     # dense fp16 MFMA flops per compute unit and clock (2.5 PFLOP/s over 256 CUs at 2.4 GHz)
REPS = 5                             # timed repetitions per leg (median reported)
UNSTABLE_SPREAD = 0.10

# Llama-3.2-1B geometry: the decode projection set the headline metric is quoted on
DIM, KV_DIM, HIDDEN, VOCAB, LAYERS = 2048, 512, 8192, 128256, 16
PREFILL_LAYERS = 4                   # distinct weight sets a prefill leg sweeps (fp16 copies: 4 x 121 MB)
# Layer copies the batched-decode and the Q4_0 / Q4_K decode legs sweep in one replayed graph: far
# more than the 256 MB memory-side cache holds (8 x 109 MB, 10 x 123 MB), and enough layers to a
# replay that the pause between two replays (a model runs 32 or more layers per replay) is a small
# part of what a layer is charged: with 3 and 4 copies the same kernels read 3-4 % slower.
BATCHED_COPIES = 8
OTHER_TYPE_COPIES = 10


class Hip:
    """The few HIP runtime calls the benchmark needs for timing: events on the context's stream."""

    def __init__(self):
        self.lib = C.CDLL("libamdhip64.so")
        self.lib.hipEventCreate.argtypes = [C.POINTER(C.c_void_p)]
        self.lib.hipEventRecord.argtypes = [C.c_void_p, C.c_void_p]
        self.lib.hipEventSynchronize.argtypes = [C.c_void_p]
        self.lib.hipEventElapsedTime.argtypes = [C.POINTER(C.c_float), C.c_void_p, C.c_void_p]
        self.lib.hipEventDestroy.argtypes = [C.c_void_p]

        self.lib.hipStreamBeginCapture.argtypes = [C.c_void_p, C.c_int]
        self.lib.hipStreamEndCapture.argtypes = [C.c_void_p, C.POINTER(C.c_void_p)]
        self.lib.hipGraphInstantiate.argtypes = [C.POINTER(C.c_void_p), C.c_void_p, C.c_void_p,
                                                 C.c_void_p, C.c_size_t]
        self.lib.hipGraphLaunch.argtypes = [C.c_void_p, C.c_void_p]
        self.lib.hipGraphExecDestroy.argtypes = [C.c_void_p]
        self.lib.hipGraphDestroy.argtypes = [C.c_void_p]
        self.lib.hipDeviceGetAttribute.argtypes = [C.POINTER(C.c_int), C.c_int, C.c_int]

    def clock_khz(self, device=0) -> int:
        """hipDeviceAttributeClockRate (enumerator 5): the device's peak shader clock."""
        v = C.c_int()
        assert self.lib.hipDeviceGetAttribute(C.byref(v), 5, device) == 0
        return int(v.value)

    def destroy_graph(self, exe):
        assert self.lib.hipGraphExecDestroy(exe) == 0

    def destroy_event(self, e):
        assert self.lib.hipEventDestroy(e) == 0

    def capture(self, stream, fn):
        """Records the kernel launches `fn` enqueues on `stream` into an executable graph."""
        assert self.lib.hipStreamBeginCapture(stream, 0) == 0
        fn()
        graph = C.c_void_p()
        assert self.lib.hipStreamEndCapture(stream, C.byref(graph)) == 0
        exe = C.c_void_p()
        assert self.lib.hipGraphInstantiate(C.byref(exe), graph, None, None, 0) == 0
        self.lib.hipGraphDestroy(graph)
        return exe

    def launch(self, exe, stream):
        assert self.lib.hipGraphLaunch(exe, stream) == 0

    def event(self):
        e = C.c_void_p()
        assert self.lib.hipEventCreate(C.byref(e)) == 0
        return e

    def record(self, e, stream):
        assert self.lib.hipEventRecord(e, stream) == 0

    def elapsed_ms(self, a, b) -> float:
        assert self.lib.hipEventSynchronize(b) == 0
        ms = C.c_float()
        assert self.lib.hipEventElapsedTime(C.byref(ms), a, b) == 0
        return float(ms.value)


def under_tracer() -> bool:
    """True when a profiler's tool library rides along (rocprofv3 preloads one)."""
    return ("rocprof" in os.environ.get("LD_PRELOAD", "").lower()
            or any(k.startswith(("ROCPROF", "ROCP_")) for k in os.environ))


def spread_stats(samples, scale=1.0, digits=4):
    """Median, range and relative spread of the repetitions."""
    med = statistics.median(samples)
    spread = (max(samples) - min(samples)) / med if med > 0 else 0.0
    return {"median": round(med * scale, digits), "min": round(min(samples) * scale, digits),
            "max": round(max(samples) * scale, digits), "spread": round(spread, 4),
            "unstable": bool(spread > UNSTABLE_SPREAD), "repetitions": len(samples)}


def timed_graph(ctx, hip, fn, steps, warmup, reps=REPS):
    """`fn`'s launches captured into one graph; `warmup` untimed replays, then `reps` repetitions
    of exactly `steps` replays between two events on the context's stream.  Returns the
    milliseconds per replay of each repetition.  The graph and the events are destroyed."""
    fn()
    ctx.sync()
    graph = hip.capture(ctx.stream, fn)
    for _ in range(warmup):
        hip.launch(graph, ctx.stream)
    ctx.sync()
    out = []
    for _ in range(reps):
        e0, e1 = hip.event(), hip.event()
        hip.record(e0, ctx.stream)
        for _ in range(steps):
            hip.launch(graph, ctx.stream)
        hip.record(e1, ctx.stream)
        out.append(hip.elapsed_ms(e0, e1) / steps)
        hip.destroy_event(e0)
        hip.destroy_event(e1)
    ctx.sync()
    hip.destroy_graph(graph)
    return out


# ---- result checks against the CPU oracle (never inside a timed region) --------------------------

def sample_rows(d, count, seed):
    """Sorted row indices: the first 16, the last 16 and a seeded random remainder."""
    rng = np.random.default_rng(seed)
    edge = np.concatenate([np.arange(min(16, d)), np.arange(max(0, d - 16), d)])
    return np.unique(np.concatenate([edge, rng.choice(d, size=min(count, d), replace=False)]))


def gather_rows(raw, t, cols, rows):
    """The blocks of the given weight rows as a small weight of its own (rows are independent)."""
    row_bytes = cols // t.block_elems * t.block_bytes
    return np.ascontiguousarray(raw.reshape(-1, row_bytes)[rows]).reshape(-1)


def oracle_rows(t, raw, cols, rows, X):
    """(reference, magnitude) of the sampled weight rows against activation rows X [B x cols]:
    the oracle's matmul in the CPU path's own summation order, and sum_j |w_ij x_bj| in float64."""
    from jitllm_amd.ggml import GGMLType
    from oracle import pyoracle as O
    sub = gather_rows(raw, t, cols, rows)
    X = np.ascontiguousarray(np.atleast_2d(X), dtype=np.float32)
    mode = O.DOT_SCALAR if t == GGMLType.Q4_K else O.DOT_VEC256
    ref = O.matmul_batch(int(t), sub, X, rows.size, cols, mode).astype(np.float64)
    w = np.abs(O.dequant(int(t), sub).reshape(rows.size, cols).astype(np.float64))
    return ref, np.abs(X.astype(np.float64)) @ w.T


def check(name, got, ref, mag, bound):
    """max |got - ref| / sum |w x| over the sample; the benchmark stops if it exceeds `bound`."""
    err = float(np.max(np.abs(np.asarray(got, dtype=np.float64) - ref) / np.maximum(mag, 1e-30)))
    if not err < bound:
        raise SystemExit(f"bench.py: {name} differs from the CPU oracle: {err:.3e} of the magnitude sum "
                         f"(bound {bound:.0e}); no figure is reported for a wrong result")
    return float(f"{err:.3e}")


def swiglu64(g, u):
    return g / (1.0 + np.exp(-g)) * u


def q8_bytes(rows, cols):
    return rows * (cols // 32) * 34


def gemv_bytes(rows, cols, block_bytes=34, block_elems=32, weights=1, outs=None):
    """Algorithmic bytes of one launch: weights + fp32 input + fp32 output."""
    outs = rows * weights if outs is None else outs
    return weights * rows * (cols // block_elems) * block_bytes + 4 * cols + 4 * outs


def build_decode_set(ctx, t):
    """Device-resident weights and activation arrays of the projection set."""
    from jitllm_amd import synthetic
    host = {
        "wq": synthetic.weight(t, DIM, DIM, 11), "wk": synthetic.weight(t, KV_DIM, DIM, 12),
        "wv": synthetic.weight(t, KV_DIM, DIM, 13), "wo": synthetic.weight(t, DIM, DIM, 14),
        "w1": synthetic.weight(t, HIDDEN, DIM, 15), "w3": synthetic.weight(t, HIDDEN, DIM, 16),
        "w2": synthetic.weight(t, DIM, HIDDEN, 17),
    }
    shapes = {"wq": (DIM, DIM), "wk": (KV_DIM, DIM), "wv": (KV_DIM, DIM), "wo": (DIM, DIM),
              "w1": (HIDDEN, DIM), "w3": (HIDDEN, DIM), "w2": (DIM, HIDDEN)}
    layers = []
    for _ in range(LAYERS):  # the same host bytes, but a device buffer of its own per layer
        layers.append({k: ctx.load_weight(t, host[k], *shapes[k]) for k in host})
    wcls_host = synthetic.weight(t, VOCAB, DIM, 18)
    wcls = ctx.load_weight(t, wcls_host, VOCAB, DIM)
    host["wcls"] = wcls_host
    shapes["wcls"] = (VOCAB, DIM)
    acts = {
        "x": ctx.from_numpy(synthetic.activations(DIM, 21)),
        "xb": ctx.from_numpy(synthetic.activations(DIM, 22)),
        "q": ctx.float_array(DIM), "k": ctx.float_array(KV_DIM), "v": ctx.float_array(KV_DIM),
        "hb": ctx.float_array(HIDDEN), "logits": ctx.float_array(VOCAB),
    }
    return layers, wcls, acts, host, shapes


def decode_step(proj, layers, wcls, acts):
    """One token's projections in the reference's decode order (LlamaQ8_0FFNLayers.java:212-525)."""
    for w in layers:
        proj.fusedQKV(acts["xb"], acts["q"], acts["k"], acts["v"], w["wq"], w["wk"], w["wv"])
        proj.residualMatvec(acts["xb"], w["wo"], DIM, DIM)
        proj.gateUp(w["w1"], w["w3"], DIM, HIDDEN)
        proj.residualMatvec(acts["hb"], w["w2"], HIDDEN, DIM)
    proj.floatMatvec(acts["xb"], acts["logits"], wcls, DIM, VOCAB)


def decode_step_fused_rms(proj, layers, wcls, acts, one_call=True):
    """The same token with the reference's fused decode kernels: the attention norm folded into
    q|k|v behind its own scale (fusedRmsNormQKVMatmulQ8), the FFN norm computed and folded inside
    gate/up (fullyFusedRmsNormFFNGateUpQ8), the final norm folded into the vocabulary projection,
    and the greedy token picked on the device (LogitsQ8_0Layer.java:85-110)."""
    for w in layers:
        proj.fusedRmsNormQKV(acts["x"], acts["q"], acts["k"], acts["v"], acts["rms_att"], None,
                             w["wq"], w["wk"], w["wv"], eps=1e-5)
        proj.residualMatvec(acts["xb"], w["wo"], DIM, DIM)
        proj.fullyFusedRmsNormGateUp(acts["x"], acts["rms_ffn"], 1e-5, w["w1"], w["w3"], DIM, HIDDEN)
        proj.residualMatvec(acts["hb"], w["w2"], HIDDEN, DIM)
    if one_call:   # the projection's workgroups keep their best logits: one launch fewer
        proj.matvecArgmax(acts["x"], acts["logits"], wcls, DIM, VOCAB, acts["token"],
                          rmsWeights=acts["rms_final"], eps=1e-5)
    else:
        proj.rmsMatvec(acts["x"], acts["rms_final"], None, acts["logits"], wcls, DIM, VOCAB, eps=1e-5)
        proj.argmax(acts["logits"], VOCAB, acts["token"])


def bench_fused_rms(ctx, hip, proj, layers, wcls, acts, host, steps, warmup):
    from jitllm_amd import synthetic
    from jitllm_amd.ggml import GGMLType
    from oracle import pyoracle as O
    rms_host = {}
    for i, k in enumerate(("rms_att", "rms_ffn", "rms_final")):
        rms_host[k] = (1.0 + 0.1 * synthetic.activations(DIM, 31 + i)).astype("float32")
        acts[k] = ctx.from_numpy(rms_host[k])
    acts["token"] = ctx.raw_buffer(4)
    # check: the vocabulary projection of the normalised vector, and the token picked from it
    x0 = acts["x"].get()
    proj.matvecArgmax(acts["x"], acts["logits"], wcls, DIM, VOCAB, acts["token"], rmsWeights=acts["rms_final"],
                      eps=1e-5)
    ctx.sync()
    logits = acts["logits"].get()
    rows = sample_rows(VOCAB, 128, 7)
    ref, mag = oracle_rows(GGMLType.Q8_0, host["wcls"], DIM, rows, O.rmsnorm(x0, rms_host["rms_final"], 1e-5))
    err = check("rms-folded vocabulary projection", logits[rows], ref[0], mag[0], 1e-3)
    if int(acts["token"].download(np.int32, 1)[0]) != int(np.argmax(logits)):
        raise SystemExit("bench.py: the device's greedy token is not the first maximum of its logits")
    ms = timed_graph(ctx, hip, lambda: decode_step_fused_rms(proj, layers, wcls, acts), steps, warmup)
    st = spread_stats(ms)
    apart = timed_graph(ctx, hip, lambda: decode_step_fused_rms(proj, layers, wcls, acts, one_call=False), steps,
                        warmup)
    return {"ms_per_step": st["median"], "ms_stats": st, "tok_s": round(1e3 / statistics.median(ms), 1),
            "launches": 4 * LAYERS + 2, "check_rel_err": err,
            "ms_per_step_with_argmax_as_its_own_scan": spread_stats(apart)["median"],
            "what": "decode set with the 33 RMS normalisations folded into q|k|v, gate/up and the "
                    "vocabulary projection (scale computed inside each kernel, no normalised vector "
                    "written) and the greedy token chosen on the device: the vocabulary projection's "
                    "workgroups keep their best logits and one small launch folds those "
                    "(ms_per_step_with_argmax_as_its_own_scan: a scan over the logits and that fold, 67 "
                    "launches)"}


def bench_short_prompt(ctx, hip, tokens, steps, warmup):
    """One Llama-3.2-1B Q8_0 layer's four batched calls between batched decode and prefill -- a
    short prompt, or the tail of a chunked one: 65 .. 511 rows, fp32 activations and the binary16
    ones the reference's prefill plan hands over, eight layers' weights swept per replay.  Checked
    against the oracle on sampled rows and columns first."""
    from jitllm_amd import synthetic
    from jitllm_amd.ggml import GGMLType
    from jitllm_amd.projections import QuantizedBatchProjections
    t, copies, bound = GGMLType.Q8_0, 8, 2e-3
    shapes = {"wq": (DIM, DIM), "wk": (KV_DIM, DIM), "wv": (KV_DIM, DIM), "wo": (DIM, DIM),
              "w1": (HIDDEN, DIM), "w3": (HIDDEN, DIM), "w2": (DIM, HIDDEN)}
    host = {k: synthetic.weight(t, r, c, 141 + i) for i, (k, (r, c)) in enumerate(shapes.items())}
    layers = [{k: ctx.load_weight(t, host[k], *shapes[k]) for k in shapes} for _ in range(copies)]
    legs = []
    for T in tokens:
        Xh = synthetic.activations((T, DIM), 148).astype(np.float16).astype(np.float32)
        Hh = (synthetic.activations((T, HIDDEN), 149) * np.float32(0.1)).astype(np.float16).astype(np.float32)
        qkv, res, hb = ctx.float_array(T * (DIM + 2 * KV_DIM)), ctx.float_array(T * DIM, fill=0.0), ctx.float_array(T * HIDDEN)
        plain = QuantizedBatchProjections(ctx, T, HIDDEN, 2 * HIDDEN)
        # (the reference's residency choice: an fp16 copy per projection kept across calls)
        keeping = QuantizedBatchProjections(ctx, T, HIDDEN, 2 * HIDDEN, resident=True)
        leg = {"tokens": T, "type": "Q8_0", "layer": "Llama-3.2-1B (dim 2048, kv 512, ffn 8192)", "layers_swept": copies}
        for name, proj, X, H in (("fp32_activations", plain, ctx.from_numpy(Xh), ctx.from_numpy(Hh)),
                                 ("fp16_activations", plain, ctx.half_from_numpy(Xh), ctx.half_from_numpy(Hh)),
                                 ("fp16_activations_resident_fp16_copy", keeping, ctx.half_from_numpy(Xh), ctx.half_from_numpy(Hh))):
            def layer(w, X=X, H=H, proj=proj):
                proj.fusedQKV(X, qkv, w["wq"], w["wk"], w["wv"])
                proj.projection(X, res, w["wo"], DIM, DIM, True)
                proj.gateUp(X, hb, w["w1"], w["w3"], DIM, HIDDEN)
                proj.projection(H, res, w["w2"], HIDDEN, DIM, True)
            res.init(0.0)
            layer(layers[0])
            ctx.sync()
            arows, ro, rh = sample_rows(T, 8, 150), sample_rows(DIM, 48, 151), sample_rows(HIDDEN, 48, 152)
            ref_o, mag_o = oracle_rows(t, host["wo"], DIM, ro, Xh[arows])
            ref_d, mag_d = oracle_rows(t, host["w2"], HIDDEN, ro, Hh[arows])
            errs = {"o+down": check(f"short prompt T={T} o + down", res.get().reshape(T, DIM)[arows][:, ro], ref_o + ref_d,
                                    mag_o + mag_d, bound)}
            g, mg = oracle_rows(t, host["w1"], DIM, rh, Xh[arows])
            u, mu = oracle_rows(t, host["w3"], DIM, rh, Xh[arows])
            errs["gate/up"] = check_swiglu(f"short prompt T={T} gate/up", hb.get().reshape(T, HIDDEN)[arows][:, rh], g, u, mg, mu, bound)
            ms = [m / copies for m in timed_graph(ctx, hip, lambda: [layer(w) for w in layers], steps, warmup)]
            med = statistics.median(ms)
            flops = 2.0 * T * (DIM * (DIM + 2 * KV_DIM) + DIM * DIM + 3 * DIM * HIDDEN)
            leg[name] = {"ms_per_layer": round(med, 4), "ms_stats": spread_stats(ms), "tok_s_per_layer": round(T / (med * 1e-3), 1),
                         "tflops": round(flops / (med * 1e-3) / 1e12, 1), "check_rel_err": errs}
        legs.append(leg)
    for w in layers:
        for tensor in w.values():
            tensor.free()
    return legs


def decode_bytes():
    """Algorithmic bytes of a step: every one of the 7 projections of a layer counted on its own
    (weight blocks + fp32 input + fp32 output), as the benchmark's definition does, even where one
    launch serves several of them."""
    per_layer = (gemv_bytes(DIM, DIM) + 2 * gemv_bytes(KV_DIM, DIM) + gemv_bytes(DIM, DIM)
                 + 2 * gemv_bytes(HIDDEN, DIM) + gemv_bytes(DIM, HIDDEN))
    return LAYERS * per_layer + gemv_bytes(VOCAB, DIM)


def cpu_timed(fn, budget_s, min_passes=3):
    """Runs `fn` once untimed, then for about `budget_s` seconds (at least `min_passes` passes);
    returns (median seconds per pass, passes, wall seconds)."""
    begin = time.perf_counter()
    fn()
    times = []
    while len(times) < min_passes or (time.perf_counter() - begin < budget_s and len(times) < 5000):
        t0 = time.perf_counter()
        fn()
        times.append(time.perf_counter() - t0)
    return statistics.median(times), len(times), time.perf_counter() - begin


def cpu_baseline(host, shapes, t, budget_s=10.0):
    """The oracle (a C restatement of FloatTensor.matmul with the 256-bit vectorDot lane order,
    rows spread over the host cores) on one layer's seven projections plus the vocabulary
    projection -- 344 MB of the 1 316 MB set -- repeated for about ``budget_s`` seconds."""
    from jitllm_amd import synthetic
    from oracle import pyoracle as O
    threads = O.max_threads()
    x_dim = synthetic.activations(DIM, 31)
    x_hid = synthetic.activations(HIDDEN, 32)
    names = ["wq", "wk", "wv", "wo", "w1", "w3", "w2", "wcls"]
    nbytes = sum(gemv_bytes(*shapes[k]) for k in names)

    def one_pass():
        for k in names:
            rows, cols = shapes[k]
            O.matmul(int(t), host[k], x_hid if cols == HIDDEN else x_dim, rows, cols, O.DOT_VEC256, threads)
    med, passes, wall = cpu_timed(one_pass, budget_s)
    return {"value": round(nbytes / med / 1e9, 2), "unit": "GB/s", "cores": threads, "kind": "port",
            "sample": f"one layer's 7 projections + vocabulary projection ({nbytes} B), "
                      f"median of {passes} passes after 1 warm-up "
                      f"({wall:.1f} s of wall time), 256-bit vectorDot order",
            "tok_s_equiv": round(nbytes / med / decode_bytes(), 3)}


def cpu_baseline_rows(t, raw, cols, rows, X, total_rows, budget_s, what):
    """The oracle's batched matmul (FloatTensor.matmul(context, ...): one dot per activation row and
    weight row, rows spread over the host cores) on a sample of a weight's rows, scaled to the
    whole weight by the row count."""
    from jitllm_amd.ggml import GGMLType
    from oracle import pyoracle as O
    threads = O.max_threads()
    sub = gather_rows(raw, t, cols, rows)
    X = np.ascontiguousarray(np.atleast_2d(X), dtype=np.float32)
    mode = O.DOT_SCALAR if t == GGMLType.Q4_K else O.DOT_VEC256
    med, passes, wall = cpu_timed(lambda: O.matmul_batch(int(t), sub, X, rows.size, cols, mode, threads), budget_s)
    flops = 2.0 * X.shape[0] * rows.size * cols
    return {"gflops": round(flops / med / 1e9, 1), "cores": threads, "kind": "port",
            "ms_whole_weight_equiv": round(med * 1e3 * total_rows / rows.size, 3),
            "sample": f"{what}: {rows.size} of {total_rows} weight rows x {X.shape[0]} activation rows, median of "
                      f"{passes} passes ({wall:.1f} s), "
                      + ("scalar dot (the type has no vector dot on the host)" if mode == O.DOT_SCALAR
                         else "256-bit vectorDot order")}


def check_swiglu(name, got, g, u, mag_g, mag_u, bound):
    """SwiGLU of two projections: the tolerance is the projections' bound carried through the
    activation (|d silu| <= 1.1 |d g|) plus, for an fp16 result, its rounding."""
    ref = swiglu64(g, u)
    mag = 1.1 * mag_g * np.abs(u) + mag_u * np.abs(g / (1.0 + np.exp(-g))) + np.abs(ref)
    return check(name, got, ref, mag, bound)


def bench_gemm(ctx, hip, t, T, steps, warmup, cpu, clock_khz, cu, dims=None, int8=True, model="Llama-3.2-1B"):
    """Batched prefill of one layer (q|k|v, o, gate/up SwiGLU, down) over T tokens: Llama-3.2-1B
    geometry unless `dims` = (dim, kv, ffn) names another; `int8` adds the block-scaled int8 mode
    (Q8_0 / Q4_0 only)."""
    from jitllm_amd import synthetic
    from jitllm_amd.projections import QuantizedBatchProjections
    DIM, KV_DIM, HIDDEN = dims or (globals()["DIM"], globals()["KV_DIM"], globals()["HIDDEN"])
    shapes = {"wq": (DIM, DIM), "wk": (KV_DIM, DIM), "wv": (KV_DIM, DIM), "wo": (DIM, DIM),
              "w1": (HIDDEN, DIM), "w3": (HIDDEN, DIM), "w2": (DIM, HIDDEN)}
    host = {k: synthetic.weight(t, r, c, 41 + i) for i, (k, (r, c)) in enumerate(shapes.items())}
    # the layer's host bytes in PREFILL_LAYERS distinct sets of device buffers, swept in turn: their
    # resident fp16 copies (121 MB a layer) together exceed the 256 MB memory-side cache, so every
    # call reads its weights from HBM as a model's successive layers do
    layers = [{k: ctx.load_weight(t, host[k], *shapes[k]) for k in shapes} for _ in range(PREFILL_LAYERS)]
    w = layers[0]
    Xh = synthetic.activations((T, DIM), 48)
    Hh = synthetic.activations((T, HIDDEN), 49) * np.float32(0.1)
    X, H = ctx.from_numpy(Xh), ctx.from_numpy(Hh)
    qkv = ctx.float_array(T * (DIM + 2 * KV_DIM))
    res = ctx.float_array(T * DIM, fill=0.0)
    hb = ctx.float_array(T * HIDDEN)
    X16, H16 = ctx.half_from_numpy(Xh), ctx.half_from_numpy(Hh)
    hb16 = ctx.half_array(T * HIDDEN)
    arows = sample_rows(T, 8, 50)          # activation rows checked
    F16_BOUND = 2e-3

    def run(proj, X=X, H=H, hb=hb, widen=False):
        def layer(w):
            proj.fusedQKV(X, qkv, w["wq"], w["wk"], w["wv"])
            proj.projection(X, res, w["wo"], DIM, DIM, True)
            proj.gateUp(X, hb, w["w1"], w["w3"], DIM, HIDDEN)
            proj.projection(H, res, w["w2"], HIDDEN, DIM, True)

        def sweep():
            for w in layers:
                layer(w)
        # result check first: q and v columns, o + down accumulated from zero, SwiGLU hidden vector
        res.init(0.0)
        layer(layers[-1])
        ctx.sync()
        xs = (Xh.astype(np.float16).astype(np.float32) if widen else Xh)[arows]
        hs = (Hh.astype(np.float16).astype(np.float32) if widen else Hh)[arows]
        errs = {}
        got = qkv.get().reshape(T, DIM + 2 * KV_DIM)[arows]
        rq, rv = sample_rows(DIM, 48, 51), sample_rows(KV_DIM, 48, 52)
        ref, mag = oracle_rows(t, host["wq"], DIM, rq, xs)
        errs["q"] = check(f"prefill T={T} q", got[:, rq], ref, mag, F16_BOUND)
        ref, mag = oracle_rows(t, host["wv"], DIM, rv, xs)
        errs["v"] = check(f"prefill T={T} v", got[:, DIM + KV_DIM + rv], ref, mag, F16_BOUND)
        ro = sample_rows(DIM, 48, 53)
        ref_o, mag_o = oracle_rows(t, host["wo"], DIM, ro, xs)
        ref_d, mag_d = oracle_rows(t, host["w2"], HIDDEN, ro, hs)
        errs["o+down"] = check(f"prefill T={T} o + down", res.get().reshape(T, DIM)[arows][:, ro], ref_o + ref_d,
                               mag_o + mag_d, F16_BOUND)
        rh = sample_rows(HIDDEN, 48, 54)
        g, mg = oracle_rows(t, host["w1"], DIM, rh, xs)
        u, mu = oracle_rows(t, host["w3"], DIM, rh, xs)
        errs["gate/up"] = check_swiglu(f"prefill T={T} gate/up", hb.get().astype(np.float32).reshape(T, HIDDEN)[arows][:, rh],
                                       g, u, mg, mu, F16_BOUND)
        # replayed as a HIP graph: Python cannot enqueue the layer's launches as fast as they run
        return [m / PREFILL_LAYERS for m in timed_graph(ctx, hip, sweep, steps, warmup)], errs

    flops = 2.0 * T * (DIM * (DIM + 2 * KV_DIM) + DIM * DIM + 2 * DIM * HIDDEN + HIDDEN * DIM)

    def mode(ms_list, errs):
        ms = statistics.median(ms_list)
        tf = flops / (ms * 1e-3) / 1e12
        return {"ms_per_layer": round(ms, 4), "ms_stats": spread_stats(ms_list), "tflops": round(tf, 1),
                "frac_f16_mfma_peak": round(tf / F16_MFMA_PEAK_TFLOPS, 4), "check_rel_err": errs}

    default = mode(*run(QuantizedBatchProjections(ctx, T, HIDDEN, 2 * HIDDEN)))
    # the reference's residency choice: an fp16 copy per projection kept across calls (2 bytes per
    # weight of HBM), decoded by the first call only -- reported beside the default, not instead
    kept = mode(*run(QuantizedBatchProjections(ctx, T, HIDDEN, 2 * HIDDEN, resident=True)))
    # the reference's own operand types on top of that: activations arrive as fp16 (its RMS apply,
    # attention and SwiGLU kernels write fp16) and the hidden vector leaves as fp16
    half_proj = QuantizedBatchProjections(ctx, T, HIDDEN, 2 * HIDDEN, resident=True)
    half = mode(*run(half_proj, X16, H16, hb16, widen=True))
    # the block-scaled int8 path (JL_MATH_INT8: activations quantised per 32-block inside the call,
    # int8 MFMA over the raw blocks, one fp32 scale product per block; Int8GemmKernels): its
    # results are fixed bit for bit, so the check is equality with the oracle's int8 statement
    from jitllm_amd import _lib as L
    from oracle import pyoracle as O
    int8_leg = None
    if int8:
        i8_proj = QuantizedBatchProjections(ctx, T, HIDDEN, 2 * HIDDEN, math=L.JL_MATH_INT8)

        def i8_layer(w=w):
            i8_proj.fusedQKV(X, qkv, w["wq"], w["wk"], w["wv"])
            i8_proj.projection(X, res, w["wo"], DIM, DIM, True)
            i8_proj.gateUp(X, hb, w["w1"], w["w3"], DIM, HIDDEN)
            i8_proj.projection(H, res, w["w2"], HIDDEN, DIM, True)

        def i8_sweep():
            for lw in layers:
                i8_layer(lw)
        res.init(0.0)
        i8_layer()
        ctx.sync()
        xq, xs = O.quantize_q8(Xh[arows])
        hq, hs = O.quantize_q8(Hh[arows])
        ro = sample_rows(DIM, 48, 56)
        ref_o = O.gemm_int8_block_scaled(int(t), xq, xs, gather_rows(host["wo"], t, DIM, ro), ro.size)
        ref_d = O.gemm_int8_block_scaled(int(t), hq, hs, gather_rows(host["w2"], t, HIDDEN, ro), ro.size)
        got = res.get().reshape(T, DIM)[arows][:, ro]
        if not np.array_equal(got.view(np.uint32), (ref_o + ref_d).astype(np.float32).view(np.uint32)):
            raise SystemExit(f"bench.py: the int8 prefill path at T={T} differs from the oracle's int8 arithmetic")
        int8_leg = mode([m / PREFILL_LAYERS for m in timed_graph(ctx, hip, i8_sweep, steps, warmup)],
                        {"o+down": "bit-equal to the oracle's int8 statement"})
        int8_leg["frac_int8_mfma_peak"] = round(int8_leg["tflops"] / INT8_MFMA_PEAK_TOPS, 4)
        int8_leg["math"] = ("int8 MFMA over the raw blocks, fp32 (float) dot * dA fused-multiplied by dW per 32-block in k order; "
                            "bound by the three vector-ALU operations per int32 result at one sixth of the int8 MFMA peak")
    # the dominant kernel on its own: the gate/up call of that last mode is one launch of the fp16
    # GEMM and nothing else (one per layer to a graph)
    def gate_ups():
        for lw in layers:
            half_proj.gateUp(X16, hb16, lw["w1"], lw["w3"], DIM, HIDDEN)
    gu = [m / PREFILL_LAYERS for m in timed_graph(ctx, hip, gate_ups, steps, 20)]
    gu_flops = 2.0 * T * 2 * HIDDEN * DIM
    gu_tf = gu_flops / (statistics.median(gu) * 1e-3) / 1e12
    peak_box = cu * clock_khz * 1e3 * F16_MFMA_FLOPS_PER_CU_CLK / 1e12
    roofline = {"bound": "mfma", "kernel": f"jl_gemm_hh gate/up SwiGLU [{T} x {DIM}] x [{2 * HIDDEN} x {DIM}]^T, fp16 in / fp16 out",
                "achieved": round(gu_tf, 1), "peak": F16_MFMA_PEAK_TFLOPS, "unit": "TFLOP/s",
                "frac": round(gu_tf / F16_MFMA_PEAK_TFLOPS, 4), "flops_per_launch": gu_flops,
                "avg_launch_us": round(statistics.median(gu) * 1e3, 2), "launch_us_stats": spread_stats(gu, 1e3, 2),
                "peak_from_box": {"compute_units": cu, "peak_clock_khz": clock_khz,
                                  "flops_per_cu_clk": F16_MFMA_FLOPS_PER_CU_CLK, "tflops": round(peak_box, 1),
                                  "frac": round(gu_tf / peak_box, 4)}}
    # what hands the projections those fp16 rows: the RMS reduction and fp16 apply of one [T x dim]
    # activation (two per layer in the model), timed on its own
    rms_w = ctx.from_numpy(np.ones(DIM, dtype=np.float32))
    rms_proj = QuantizedBatchProjections(ctx, T, DIM, DIM)
    def rms_apply():
        # (8 launches per graph: a one-kernel graph measures the graph launch, not the kernel)
        for _ in range(8):
            rms_proj.rmsApplyFP16(X, rms_w, 1e-5, X16, DIM)
    rms_us = statistics.median(timed_graph(ctx, hip, rms_apply, steps, 3)) / 8 * 1e3
    half["rms_apply_to_fp16_us"] = round(rms_us, 2)
    copy_mb = round(2e-6 * sum(r * c for r, c in shapes.values()))
    out = {"tokens": T, "type": t.name, "layer": f"{model} (dim {DIM}, kv {KV_DIM}, ffn {HIDDEN})",
           "layers_swept": PREFILL_LAYERS,
           "weights_from": f"HBM: {PREFILL_LAYERS} layers' distinct weights in turn (their fp16 copies, "
                           f"{PREFILL_LAYERS} x {copy_mb} MB, exceed the 256 MB memory-side cache)",
           "ms_per_layer": default["ms_per_layer"],
           "ms_stats": default["ms_stats"],
           "tok_s_per_layer": round(T / (default["ms_per_layer"] * 1e-3), 1),
           "tflops": default["tflops"], "frac_f16_mfma_peak": default["frac_f16_mfma_peak"],
           "check_rel_err": default["check_rel_err"],
           "math": "f16 MFMA, fp32 accumulate; weights decoded to fp16 inside the call (in LDS, or once per call into the workspace)",
           "with_resident_fp16_copy": kept, "with_resident_copy_and_fp16_activations": half,
           "roofline": roofline}
    if dims is None:
        out["tok_s_16_layers"] = round(T / (default["ms_per_layer"] * 1e-3 * LAYERS), 1)
    if int8_leg is not None:
        out["int8_block_scaled"] = int8_leg
    if cpu:
        rows = sample_rows(HIDDEN, 224, 55)
        out["cpu_baseline"] = cpu_baseline_rows(t, host["w1"], DIM, rows, Xh, HIDDEN, 2.0, f"gate projection at T={T}")
        out["cpu_baseline"]["ms_per_layer_equiv"] = round(
            flops / (out["cpu_baseline"]["gflops"] * 1e9) * 1e3, 1)
    for lw in layers:
        for x in lw.values():
            x.free()
    return out


def bench_batched(ctx, hip, B, steps, warmup, cpu, type_name="Q4_K", dims=(4096, 1024, 12288),
                  model="Qwen3-8B-like", copies=None):
    """Batched decode of one layer's projections for B sequences: Q4_K at Qwen3-8B-like shapes (dim
    4096, ffn 12288, kv 1024) unless another type and geometry are named."""
    from jitllm_amd import synthetic
    from jitllm_amd.ggml import GGMLType
    from jitllm_amd.projections import QuantizedBatchProjections
    t = GGMLType[type_name]
    dim, kv, ffn = dims
    shapes = {"wq": (dim, dim), "wk": (kv, dim), "wv": (kv, dim), "wo": (dim, dim),
              "w1": (ffn, dim), "w3": (ffn, dim), "w2": (dim, ffn)}
    host = {k: synthetic.weight(t, r, c, 61 + i) for i, (k, (r, c)) in enumerate(shapes.items())}
    # enough copies of the layer (109 MB each) that a replay cannot be served from the 256 MB
    # memory-side cache, whatever it keeps of what it has seen
    copies = copies or BATCHED_COPIES
    layers = [{k: ctx.load_weight(t, host[k], *shapes[k]) for k in shapes} for _ in range(copies)]
    Xh = synthetic.activations((B, dim), 68)
    Hh = synthetic.activations((B, ffn), 69) * np.float32(0.1)
    X, H = ctx.from_numpy(Xh), ctx.from_numpy(Hh)
    qkv = ctx.float_array(B * (dim + 2 * kv))
    res = ctx.float_array(B * dim, fill=0.0)
    hb = ctx.float_array(B * ffn)
    proj = QuantizedBatchProjections(ctx, B, ffn, 2 * ffn)

    def layer(w):
        proj.fusedQKV(X, qkv, w["wq"], w["wk"], w["wv"])
        proj.projection(X, res, w["wo"], dim, dim, True)
        proj.gateUp(X, hb, w["w1"], w["w3"], dim, ffn)
        proj.projection(H, res, w["w2"], ffn, dim, True)

    layer(layers[0])
    ctx.sync()
    errs = {}
    got = qkv.get().reshape(B, dim + 2 * kv)
    rq, rk = sample_rows(dim, 32, 71), sample_rows(kv, 32, 72)
    ref, mag = oracle_rows(t, host["wq"], dim, rq, Xh)
    errs["q"] = check(f"batched B={B} q", got[:, rq], ref, mag, 2e-3)
    ref, mag = oracle_rows(t, host["wk"], dim, rk, Xh)
    errs["k"] = check(f"batched B={B} k", got[:, dim + rk], ref, mag, 2e-3)
    ro = sample_rows(dim, 32, 73)
    ref_o, mag_o = oracle_rows(t, host["wo"], dim, ro, Xh)
    ref_d, mag_d = oracle_rows(t, host["w2"], ffn, ro, Hh)
    errs["o+down"] = check(f"batched B={B} o + down", res.get().reshape(B, dim)[:, ro], ref_o + ref_d,
                           mag_o + mag_d, 2e-3)
    rh = sample_rows(ffn, 32, 74)
    g, mg = oracle_rows(t, host["w1"], dim, rh, Xh)
    u, mu = oracle_rows(t, host["w3"], dim, rh, Xh)
    errs["gate/up"] = check_swiglu(f"batched B={B} gate/up", hb.get().reshape(B, ffn)[:, rh], g, u, mg, mu, 2e-3)

    def sweep():
        for w in layers:
            layer(w)
    ms_list = [m / copies for m in timed_graph(ctx, hip, sweep, steps, warmup)]
    ms = statistics.median(ms_list)
    wbytes = sum(a.size for a in host.values())
    # fp32 activations in and out, once per projection
    io = 4 * B * (dim + dim + 2 * kv + dim + dim + dim + ffn + ffn + dim)
    flops = 2.0 * B * (dim * (dim + 2 * kv) + dim * dim + 2 * dim * ffn + ffn * dim)
    gbs = (wbytes + io) / (ms * 1e-3) / 1e9
    out = {"B": B, "type": type_name, "layer": f"{model} (dim {dim}, kv {kv}, ffn {ffn})",
           "ms_per_layer": round(ms, 4), "ms_stats": spread_stats(ms_list), "layers_swept": copies,
           "GB_s": round(gbs, 1), "frac_hbm_peak": round(gbs / HBM_PEAK_GBS, 4),
           "tflops": round(flops / (ms * 1e-3) / 1e12, 1), "bytes": wbytes + io, "check_rel_err": errs}
    # which roof applies at this batch: the call's flop per byte against the chip's ridge
    intensity = flops / (wbytes + io)
    ridge = F16_MFMA_PEAK_TFLOPS * 1e12 / (HBM_PEAK_GBS * 1e9)
    out["flop_per_byte"] = round(intensity, 1)
    out["bound"] = "hbm" if intensity < ridge else "mfma"
    out["frac_f16_mfma_peak"] = round(out["tflops"] / F16_MFMA_PEAK_TFLOPS, 4)
    if cpu and B == 8:
        rows = sample_rows(ffn, 480 if t == GGMLType.Q4_K else 2048, 75)
        out["cpu_baseline"] = cpu_baseline_rows(t, host["w1"], dim, rows, Xh, ffn, 2.0, "gate projection at B=8")
        out["cpu_baseline"]["ms_per_layer_equiv"] = round(flops / (out["cpu_baseline"]["gflops"] * 1e9) * 1e3, 1)
    for w in layers:
        for x in w.values():
            x.free()
    return out


def bench_batched_vocabulary(ctx, hip, type_name, vocab, dim, model, rows_list, steps, warmup):
    """The vocabulary projection of a batched decode step -- logits for B sequences -- over two copies
    of the weight in turn (each larger than the 256 MB memory-side cache): the weight-streaming kernel
    on a launch large enough that its fixed costs are a small part."""
    from jitllm_amd import synthetic
    from jitllm_amd.ggml import GGMLType
    from jitllm_amd.projections import QuantizedBatchProjections
    t = GGMLType[type_name]
    host = synthetic.weight(t, vocab, dim, 91)
    ws = [ctx.load_weight(t, host, vocab, dim) for _ in range(2)]
    legs = []
    for B in rows_list:
        Xh = synthetic.activations((B, dim), 92 + B)
        X, out = ctx.from_numpy(Xh), ctx.float_array(B * vocab)
        proj = QuantizedBatchProjections(ctx, B, dim, vocab)
        proj.projection(X, out, ws[0], dim, vocab, False)
        ctx.sync()
        rows = sample_rows(vocab, 64, 93)
        ref, mag = oracle_rows(t, host, dim, rows, Xh)
        err = check(f"batched vocabulary projection B={B}", out.get().reshape(B, vocab)[:, rows], ref, mag, 2e-3)

        def sweep():      # (sixteen calls to a replay: the pause between replays is shared)
            for _ in range(8):
                for w in ws:
                    proj.projection(X, out, w, dim, vocab, False)
        us_list = [m / (8 * len(ws)) * 1e3 for m in timed_graph(ctx, hip, sweep, steps, warmup)]
        us = statistics.median(us_list)
        nbytes = host.size + 4 * B * (dim + vocab)
        # ... and the greedy token of every row (batchedArgmaxLogits), one launch over the B x vocab logits
        tokens = ctx.raw_buffer(4 * B)
        proj.argmaxLogits(out, vocab, tokens)
        ctx.sync()
        if not np.array_equal(tokens.download(np.int32, B), np.argmax(out.get().reshape(B, vocab), axis=1)):
            raise SystemExit("bench.py: the device's per-row greedy tokens are not the first maxima of its logits")

        def picks():
            for _ in range(16):
                proj.argmaxLogits(out, vocab, tokens)
        argmax_us = statistics.median(m / 16 * 1e3 for m in timed_graph(ctx, hip, picks, steps, warmup))
        legs.append({"B": B, "us_per_call": round(us, 2), "us_stats": spread_stats(us_list), "bytes": nbytes,
                     "GB_s": round(nbytes / us / 1e3, 1), "frac_hbm_peak": round(nbytes / us / 1e3 / HBM_PEAK_GBS, 4),
                     "check_rel_err": err, "argmax_rows_us": round(argmax_us, 2)})
        for b in (X, out, proj.workspace, tokens):
            b.free()
    for w in ws:
        w.free()
    return {"type": type_name, "weight": f"{model} vocabulary projection [{vocab} x {dim}]", "weight_bytes": int(host.size),
            "copies_swept": len(ws), "rows": legs}


def bench_decode_layers(ctx, hip, type_name, dim, kv, ffn, copies, steps, warmup, cpu):
    """Single-token decode projections of one layer -- q|k|v, o (+=), gate/up SwiGLU, down (+=) --
    over `copies` distinct layers' weights (more bytes than the 256 MB last-level cache holds),
    replayed as one HIP graph.  Q4_0 at Llama-3-8B shapes and Q4_K at Qwen3-8B-like shapes: the
    other two weight types the path is specified on.  Timed twice: the fp32-activation path (the one
    held to the CPU path's results) and the reference's optional packed-integer path, whose four
    activation quantisations per layer are launches of their own here and are counted."""
    from jitllm_amd import synthetic
    from jitllm_amd.ggml import GGMLType
    from jitllm_amd.projections import PackedActivation, QuantizedProjections, TornadoWorkspace
    from oracle import pyoracle as O
    t = GGMLType[type_name]
    shapes = {"wq": (dim, dim), "wk": (kv, dim), "wv": (kv, dim), "wo": (dim, dim),
              "w1": (ffn, dim), "w3": (ffn, dim), "w2": (dim, ffn)}
    host = {k: synthetic.weight(t, r, c, 71 + i) for i, (k, (r, c)) in enumerate(shapes.items())}
    layers = [{k: ctx.load_weight(t, host[k], *shapes[k]) for k in shapes} for _ in range(copies)]
    xh, xbh = synthetic.activations(dim, 78), synthetic.activations(dim, 79)
    hbh = synthetic.activations(ffn, 80) * np.float32(0.1)
    x, xb = ctx.from_numpy(xh), ctx.from_numpy(xbh)
    q, k_, v = ctx.float_array(dim), ctx.float_array(kv), ctx.float_array(kv)
    hb = ctx.from_numpy(hbh)
    hb2 = ctx.float_array(ffn)
    proj = QuantizedProjections(ctx, TornadoWorkspace(wrapX=x, wrapXb=xb, wrapHb=hb2, wrapHb2=hb))
    small = QuantizedProjections(ctx, TornadoWorkspace(wrapHb=hb2, packedX=PackedActivation(ctx, dim)), packed=True)
    wide = QuantizedProjections(ctx, TornadoWorkspace(packedX=PackedActivation(ctx, ffn)), packed=True)

    def layer(w):
        proj.fusedQKV(xb, q, k_, v, w["wq"], w["wk"], w["wv"])
        proj.residualMatvec(xb, w["wo"], dim, dim)
        proj.gateUp(w["w1"], w["w3"], dim, ffn)
        proj.residualMatvec(hb, w["w2"], ffn, dim)

    def step():
        for w in layers:
            layer(w)

    def step_packed():
        for w in layers:
            small.quantize(xb, dim)
            small.packedFusedQKV(q, k_, v, w["wq"], w["wk"], w["wv"])
            small.quantize(xb, dim)                      # the attention output
            small.packedMatvec(x, w["wo"], dim, dim, residual=True)
            small.quantize(xb, dim)                      # the feed-forward input
            small.packedGateUp(w["w1"], w["w3"], dim, ffn)
            wide.quantize(hb, ffn)
            wide.packedMatvec(x, w["w2"], ffn, dim, residual=True)

    # check one layer of the fp32-activation path: q, the two residual projections, gate/up
    layer(layers[0])
    ctx.sync()
    errs = {}
    rq, ro, rh = sample_rows(dim, 64, 81), sample_rows(dim, 64, 82), sample_rows(ffn, 64, 83)
    ref, mag = oracle_rows(t, host["wq"], dim, rq, xbh)
    errs["q"] = check(f"{type_name} decode q", q.get()[rq], ref[0], mag[0], 1e-3)
    ref_o, mag_o = oracle_rows(t, host["wo"], dim, ro, xbh)
    ref_d, mag_d = oracle_rows(t, host["w2"], ffn, ro, hbh)
    errs["o+down"] = check(f"{type_name} decode o + down", x.get()[ro] - xh[ro].astype(np.float64), (ref_o + ref_d)[0],
                           (mag_o + mag_d + np.abs(xh[ro]) * 1e-6)[0], 1e-3)
    g, mg = oracle_rows(t, host["w1"], dim, rh, xbh)
    u, mu = oracle_rows(t, host["w3"], dim, rh, xbh)
    errs["gate/up"] = check_swiglu(f"{type_name} decode gate/up", hb2.get()[rh], g[0], u[0], mg[0], mu[0], 1e-3)

    ms_list = [m / copies for m in timed_graph(ctx, hip, step, steps, warmup)]
    packed_list = [m / copies for m in timed_graph(ctx, hip, step_packed, steps, warmup)]
    ms, ms_packed = statistics.median(ms_list), statistics.median(packed_list)
    wbytes = sum(a.size for a in host.values())
    io = 4 * (dim + dim + 2 * kv + dim + dim + dim + ffn + ffn + dim)
    gbs = (wbytes + io) / (ms * 1e-3) / 1e9
    out = {"type": type_name, "shapes": {"dim": dim, "kv": kv, "ffn": ffn}, "layers_swept": copies,
           "ms_per_layer": round(ms, 4), "ms_stats": spread_stats(ms_list), "GB_s": round(gbs, 1),
           "frac_hbm_peak": round(gbs / HBM_PEAK_GBS, 4), "bytes_per_layer": wbytes + io, "check_rel_err": errs,
           "packed_activation_path": {"ms_per_layer": round(ms_packed, 4), "ms_stats": spread_stats(packed_list),
                                      "launches_per_layer": 8,
                                      "GB_s": round((wbytes + io) / (ms_packed * 1e-3) / 1e9, 1)}}
    if cpu:
        threads = O.max_threads()
        mode = O.DOT_SCALAR if t == GGMLType.Q4_K else O.DOT_VEC256

        def one_pass():
            for name, (r, c) in shapes.items():
                O.matmul(int(t), host[name], hbh if c == ffn else xbh, r, c, mode, threads)
        med, passes, wall = cpu_timed(one_pass, 2.0)
        out["cpu_baseline"] = {"value": round((wbytes + io) / med / 1e9, 2), "unit": "GB/s", "cores": threads,
                               "kind": "port",
                               "sample": f"the layer's 7 projections ({wbytes + io} B), median of {passes} passes "
                                         f"({wall:.1f} s), "
                                         + ("scalar dot" if mode == O.DOT_SCALAR else "256-bit vectorDot order")}
    for w in layers:
        for a in w.values():
            a.free()
    return out


def bench_wq_shape(ctx, hip, t, steps, warmup, cpu):
    """The single 2048 x 2048 Q8_0 projection (Llama-3.2-1B wq), two ways: *hot* -- the same weight
    replayed, 4.5 MB that stay in the L2 / memory-side cache, labelled as such -- and *cold* --
    rotating over 96 device copies (428 MB, more than the 256 MB memory-side cache holds), the
    model-free form of the reference's SyntheticKernelBench."""
    from jitllm_amd import synthetic
    from jitllm_amd.projections import QuantizedProjections, TornadoWorkspace
    from oracle import pyoracle as O
    raw = synthetic.weight(t, DIM, DIM, 11)
    xh = synthetic.activations(DIM, 21)
    copies = [ctx.load_weight(t, raw, DIM, DIM) for _ in range(96)]
    x, out = ctx.from_numpy(xh), ctx.float_array(DIM)
    proj = QuantizedProjections(ctx, TornadoWorkspace())
    proj.floatMatvec(x, out, copies[-1], DIM, DIM)
    ctx.sync()
    rows = sample_rows(DIM, 256, 9)
    ref, mag = oracle_rows(t, raw, DIM, rows, xh)
    err = check("2048 x 2048 projection", out.get()[rows], ref[0], mag[0], 1e-3)

    def hot():
        for _ in range(96):
            proj.floatMatvec(x, out, copies[0], DIM, DIM)

    def cold():
        for w in copies:
            proj.floatMatvec(x, out, w, DIM, DIM)
    nbytes = gemv_bytes(DIM, DIM)
    res = {"shape": "Q8_0 [2048 x 2048], batch 1", "bytes_per_launch": nbytes, "check_rel_err": err}
    for name, fn, note in (("hot", hot, "same weight every launch: served from L2 / the memory-side cache, not HBM"),
                           ("cold_rotating", cold, "96 device copies in turn (428 MB): every launch reads HBM")):
        us = [m / 96 * 1e3 for m in timed_graph(ctx, hip, fn, steps, warmup)]
        med = statistics.median(us)
        res[name] = {"us_per_launch": round(med, 3), "us_stats": spread_stats(us, 1.0, 3),
                     "GB_s": round(nbytes / med / 1e3, 1), "frac_hbm_peak": round(nbytes / med / 1e3 / HBM_PEAK_GBS, 4),
                     "note": note}
    if cpu:
        threads = O.max_threads()
        med, passes, wall = cpu_timed(lambda: O.matmul(int(t), raw, xh, DIM, DIM, O.DOT_VEC256, threads), 1.0)
        res["cpu_baseline"] = {"value": round(nbytes / med / 1e9, 2), "unit": "GB/s", "cores": threads, "kind": "port",
                               "sample": f"the same projection, median of {passes} passes ({wall:.1f} s), host caches warm"}
    for w in copies:
        w.free()
    return res


# HBM bytes one gate/up launch moves, from `rocprofv3 --pmc FETCH_SIZE` and `--pmc WRITE_SIZE` over
# `bench.py --traffic-probe` (profiles/gemv_q8_0_gate_up_hbm_traffic.md): 17 475 KiB x 2.0 read
# (the counter books 64 bytes for each of this chip's 128-byte requests; a 256 MiB plain copy reads
# 131 087 KiB on it) + 64 KiB x 1.0 written.  The algorithmic figure is 35 733 504 bytes.
GATE_UP_HBM_TRAFFIC_BYTES = 17475 * 1024 * 2 + 64 * 1024


def traffic_probe(ctx, proj, layers):
    """What `rocprofv3 --pmc FETCH_SIZE` / `--pmc WRITE_SIZE` are collected on.

    Launches, kernel by kernel (no graph, so every dispatch has a counter row of its own):
      1. the calibration kernel: a plain device-to-device copy of 256 MiB of floats (torch's
         elementwise copy kernel), which reads 268 435 456 bytes once and writes as many, so the
         counters' units and the size of the memory requests they count can be read off a
         transfer of known size;
      2. the fused gate/up GEMV of each of the 16 layers (distinct weights, 35 651 584 bytes each),
         three rounds.
    Prints the byte counts the counter values are to be compared with.
    """
    import torch
    src = torch.ones(64 * 1024 * 1024, dtype=torch.float32, device="cuda:0")
    dst = torch.empty_like(src)
    for _ in range(3):
        dst.copy_(src)
    torch.cuda.synchronize()
    for _ in range(3):
        for w in layers:
            proj.gateUp(w["w1"], w["w3"], DIM, HIDDEN)
    ctx.sync()
    print(json.dumps({"calibration": {"kernel": "torch copy_ of 64 Mi floats",
                                      "read_bytes": src.numel() * 4, "write_bytes": src.numel() * 4},
                      "gate_up": {"algorithmic_read_bytes": 2 * gemv_bytes(HIDDEN, DIM) + 4 * DIM,
                                  "algorithmic_write_bytes": 4 * HIDDEN}}))


def roofline_probe(ctx, hip, proj, layers, replays=12):
    """What the kernel trace behind `roofline.avg_launch_us` is collected on: the fused gate/up GEMV
    launched the way the benchmark's roofline leg launches it -- one HIP graph of four sweeps over
    the 16 layers' distinct weights, 64 launches back to back, replayed `replays` times -- so that
    the tracer's per-dispatch durations are of launches that follow one another as in the timed
    leg, not of launches enqueued one by one from Python.  Prints the HIP-event figure of the same
    replays (what the benchmark itself reports) beside the launch count the trace must hold."""
    def sweeps():
        for _ in range(4):
            for w in layers:
                proj.gateUp(w["w1"], w["w3"], DIM, HIDDEN)
    us = [m / (4 * LAYERS) * 1e3 for m in timed_graph(ctx, hip, sweeps, replays, 2, reps=3)]
    print(json.dumps({"roofline_probe": {"kernel": "gate/up GEMV 2 x [8192 x 2048]", "launches_per_replay": 4 * LAYERS,
                                         "replays": 2 + 3 * replays, "launches_outside_graph": 4 * LAYERS,
                                         "bytes_per_launch": 2 * gemv_bytes(HIDDEN, DIM),
                                         "hip_event_us_per_launch": spread_stats(us, 1.0, 3)}}))


def decode_probe(ctx, proj, layers, wcls, acts):
    """What the kernel trace of the decode kernels is collected on: the 65 launches of a decode
    step, kernel by kernel (no graph: a tracer serialises a replayed graph anyway), six steps over
    the 16 layers' distinct weights; then one layer at 8B-model shapes for the other two weight
    types (Q4_0: ffn 14336, Q4_K: ffn 12288), five device copies in turn, four rounds."""
    from jitllm_amd import synthetic
    from jitllm_amd.ggml import GGMLType
    from jitllm_amd.projections import QuantizedProjections, TornadoWorkspace
    for _ in range(6):
        decode_step(proj, layers, wcls, acts)
    ctx.sync()
    dim, kv = 4096, 1024
    for type_name, ffn in (("Q4_0", 14336), ("Q4_K", 12288)):
        t = GGMLType[type_name]
        shapes = {"wq": (dim, dim), "wk": (kv, dim), "wv": (kv, dim), "wo": (dim, dim),
                  "w1": (ffn, dim), "w3": (ffn, dim), "w2": (dim, ffn)}
        host = {k: synthetic.weight(t, r, c, 71 + i) for i, (k, (r, c)) in enumerate(shapes.items())}
        copies = [{k: ctx.load_weight(t, host[k], *shapes[k]) for k in shapes} for _ in range(5)]
        x, xb = ctx.from_numpy(synthetic.activations(dim, 78)), ctx.from_numpy(synthetic.activations(dim, 79))
        q, k_, v = ctx.float_array(dim), ctx.float_array(kv), ctx.float_array(kv)
        hb = ctx.from_numpy(synthetic.activations(ffn, 80) * np.float32(0.1))
        hb2 = ctx.float_array(ffn)
        p8 = QuantizedProjections(ctx, TornadoWorkspace(wrapX=x, wrapXb=xb, wrapHb=hb2, wrapHb2=hb))
        for _ in range(4):
            for w in copies:
                p8.fusedQKV(xb, q, k_, v, w["wq"], w["wk"], w["wv"])
                p8.residualMatvec(xb, w["wo"], dim, dim)
                p8.gateUp(w["w1"], w["w3"], dim, ffn)
                p8.residualMatvec(hb, w["w2"], ffn, dim)
        ctx.sync()
        for w in copies:
            for a in w.values():
                a.free()
    print(json.dumps({"decode_probe": {"steps": 6, "launches_per_step": 65,
                                       "other_types": {"layers": 5, "rounds": 4}}}))


def prefill_probe(ctx, t, T=2048, mode="xf16"):
    """What the matrix-pipe counters (`rocprofv3 --pmc SQ_INSTS_VALU_MFMA_MOPS_F16 SQ_VALU_MFMA_BUSY_CYCLES
    SQ_BUSY_CU_CYCLES GRBM_GUI_ACTIVE`) and the prefill kernel traces are collected on: one
    Llama-3.2-1B layer's four prefill calls at T tokens over PREFILL_LAYERS distinct sets of weights
    in turn (so that they are read from HBM), launched kernel by kernel -- no graph, so that every
    dispatch has a row of its own -- four passes.  Mode "xf16": resident fp16 copy and fp16
    activations (every call is then one launch of the fp16 GEMM, plus a fold where K is cut; the first
    pass decodes the copy); "resident": the copy with fp32 activations; "default": plain `jl_gemm`."""
    from jitllm_amd import synthetic
    from jitllm_amd.projections import QuantizedBatchProjections
    shapes = {"wq": (DIM, DIM), "wk": (KV_DIM, DIM), "wv": (KV_DIM, DIM), "wo": (DIM, DIM),
              "w1": (HIDDEN, DIM), "w3": (HIDDEN, DIM), "w2": (DIM, HIDDEN)}
    host = {k: synthetic.weight(t, r, c, 41 + i) for i, (k, (r, c)) in enumerate(shapes.items())}
    layers = [{k: ctx.load_weight(t, host[k], *shapes[k]) for k in shapes} for _ in range(PREFILL_LAYERS)]
    x_host = synthetic.activations((T, DIM), 48)
    h_host = synthetic.activations((T, HIDDEN), 49) * np.float32(0.1)
    qkv, res = ctx.float_array(T * (DIM + 2 * KV_DIM)), ctx.float_array(T * DIM, fill=0.0)
    if mode == "xf16":
        x, h, hb = ctx.half_from_numpy(x_host), ctx.half_from_numpy(h_host), ctx.half_array(T * HIDDEN)
    else:
        x, h, hb = ctx.from_numpy(x_host), ctx.from_numpy(h_host), ctx.float_array(T * HIDDEN)
    proj = QuantizedBatchProjections(ctx, T, HIDDEN, 2 * HIDDEN, resident=mode != "default")
    for _ in range(4):
        for w in layers:
            proj.fusedQKV(x, qkv, w["wq"], w["wk"], w["wv"])
            proj.projection(x, res, w["wo"], DIM, DIM, True)
            proj.gateUp(x, hb, w["w1"], w["w3"], DIM, HIDDEN)
            proj.projection(h, res, w["w2"], HIDDEN, DIM, True)
        ctx.sync()
    print(json.dumps({"tokens": T, "mode": mode, "layers_swept": PREFILL_LAYERS, "passes": 4, "flops": {"q|k|v": 2.0 * T * DIM * (DIM + 2 * KV_DIM), "o": 2.0 * T * DIM * DIM,
                                             "gate/up": 2.0 * T * 2 * HIDDEN * DIM, "down": 2.0 * T * HIDDEN * DIM},
                      "mfma_f16_flops_per_instruction_16x16x32": 2 * 16 * 16 * 32}))


def _probes_lib():
    lib = C.CDLL(os.path.join(os.path.dirname(os.path.abspath(__file__)), "jitllm_amd", "lib", "libjl_probes.so"))
    lib.jl_probe_mfma_rate.argtypes = [C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, C.POINTER(C.c_double)]
    lib.jl_probe_mfma_rate.restype = C.c_int
    lib.jl_probe_hbm_read_rate.argtypes = [C.c_int, C.c_size_t, C.c_int, C.c_int, C.POINTER(C.c_double)]
    lib.jl_probe_hbm_read_rate.restype = C.c_int
    return lib


def hbm_rate_probe(cu, reps=5, gib=2):
    """The rate at which the chip streams HBM with nothing else in the way, measured by
    `jitllm_amd/lib/libjl_probes.so` (a measurement aid built beside the product library, not part
    of it): plain 16-byte loads over `gib` GiB (far more than the 256 MB memory-side cache), eight
    in flight per thread, 8 workgroups of 256 per compute unit.  Median of `reps` launches, the
    first left out.  The decode kernels' fractions of the published 8 TB/s are to be read against it."""
    buf = (C.c_double * (reps + 1))()
    rc = _probes_lib().jl_probe_hbm_read_rate(0, gib << 30, reps + 1, cu, buf)
    if rc != 0:
        raise RuntimeError(f"jl_probe_hbm_read_rate: HIP error {rc}")
    return {"what": f"plain streaming read of {gib} GiB, GB/s (median of {reps} launches)",
            "hbm_read_GB_s": round(statistics.median(list(buf)[1:]), 1)}


def mfma_rate_probe(cu, reps=5, steps=20000):
    """The rate at which the chip sustains fp16 matrix instructions out of registers, measured by
    `jitllm_amd/lib/libjl_probes.so` (a measurement aid built beside the product library, not part
    of it): loops of nothing but `v_mfma_f32_16x16x32_f16` / `32x32x16` on one 8-wave workgroup per
    compute unit, with every operand 1.0 and with random operands.  The published 2.5 PFLOP/s is
    reached only by the former; the latter is what a GEMM on real data can approach.  Medians over
    `reps` launches of about 20 ms, the first left out (the clock settles during it)."""
    lib = _probes_lib()
    out = {"what": "register-only MFMA loops, 8 waves per compute unit, TFLOP/s (median of %d launches)" % reps}
    for shape, name in ((0, "16x16x32"), (1, "32x32x16")):
        for random, data in ((1, "random_operands"), (0, "constant_operands")):
            buf = (C.c_double * (reps + 1))()
            rc = lib.jl_probe_mfma_rate(0, shape, random, steps, reps + 1, cu, buf)
            if rc != 0:
                raise RuntimeError(f"jl_probe_mfma_rate: HIP error {rc}")
            out[f"{name}_{data}"] = round(statistics.median(list(buf)[1:]), 1)
    return out


def batched_probe(ctx):
    """What the kernel trace of the batched-decode kernels is collected on: the four calls of one
    Q4_K Qwen3-8B-like layer (q|k|v, o +=, gate/up SwiGLU, down +=) at 8, 32 and 64 rows, launched
    kernel by kernel over three device copies of the layer in turn (325 MB, more than the
    memory-side cache holds), four rounds each."""
    from jitllm_amd import synthetic
    from jitllm_amd.ggml import GGMLType
    from jitllm_amd.projections import QuantizedBatchProjections
    t = GGMLType.Q4_K
    dim, kv, ffn = 4096, 1024, 12288
    shapes = {"wq": (dim, dim), "wk": (kv, dim), "wv": (kv, dim), "wo": (dim, dim),
              "w1": (ffn, dim), "w3": (ffn, dim), "w2": (dim, ffn)}
    host = {k: synthetic.weight(t, r, c, 61 + i) for i, (k, (r, c)) in enumerate(shapes.items())}
    layers = [{k: ctx.load_weight(t, host[k], *shapes[k]) for k in shapes} for _ in range(3)]
    for B in (8, 32, 64):
        X = ctx.from_numpy(synthetic.activations((B, dim), 68))
        H = ctx.from_numpy(synthetic.activations((B, ffn), 69) * np.float32(0.1))
        qkv, res, hb = ctx.float_array(B * (dim + 2 * kv)), ctx.float_array(B * dim, fill=0.0), ctx.float_array(B * ffn)
        proj = QuantizedBatchProjections(ctx, B, ffn, 2 * ffn)
        for _ in range(4):
            for w in layers:
                proj.fusedQKV(X, qkv, w["wq"], w["wk"], w["wv"])
                proj.projection(X, res, w["wo"], dim, dim, True)
                proj.gateUp(X, hb, w["w1"], w["w3"], dim, ffn)
                proj.projection(H, res, w["w2"], ffn, dim, True)
            ctx.sync()
    print(json.dumps({"weight_bytes": {k: int(v.size) for k, v in host.items()}}))


def vocabulary_probe(ctx):
    """What the kernel trace of the batched vocabulary projection is collected on: the Q8_0
    [128256 x 2048] projection and the per-row greedy token at 8, 32 and 64 rows, kernel by kernel
    over two device copies of the weight in turn, six rounds each."""
    from jitllm_amd import synthetic
    from jitllm_amd.ggml import GGMLType
    from jitllm_amd.projections import QuantizedBatchProjections
    t = GGMLType.Q8_0
    host = synthetic.weight(t, VOCAB, DIM, 91)
    ws = [ctx.load_weight(t, host, VOCAB, DIM) for _ in range(2)]
    for B in (8, 32, 64):
        X, out = ctx.from_numpy(synthetic.activations((B, DIM), 92 + B)), ctx.float_array(B * VOCAB)
        tokens = ctx.raw_buffer(4 * B)
        proj = QuantizedBatchProjections(ctx, B, DIM, VOCAB)
        for _ in range(6):
            for w in ws:
                proj.projection(X, out, w, DIM, VOCAB, False)
                proj.argmaxLogits(out, VOCAB, tokens)
            ctx.sync()
    print(json.dumps({"weight_bytes": int(host.size)}))


def shapes_probe(ctx):
    """What the kernel trace of the shapes beside the benchmark's is collected on: single-token
    projections over rows longer than 16 384 columns (the two-halves form of the tile kernel) and batched
    decode over rows whose blocks have no cut into equal spans (two column windows), each beside a
    well-shaped neighbour, kernel by kernel over three device copies in turn, four rounds each."""
    from jitllm_amd import synthetic
    from jitllm_amd.ggml import GGMLType
    from jitllm_amd.projections import QuantizedBatchProjections, QuantizedProjections, TornadoWorkspace
    shapes = {}
    for name, d, n in (("Q8_0", 5120, 16384), ("Q8_0", 5120, 17408), ("Q4_K", 5120, 27648), ("Q4_0", 8192, 28672)):
        t = GGMLType[name]
        host = synthetic.weight(t, d, n, 95)
        ws = [ctx.load_weight(t, host, d, n) for _ in range(3)]
        proj = QuantizedProjections(ctx, TornadoWorkspace())
        x, out = ctx.from_numpy(synthetic.activations(n, 96)), ctx.float_array(d)
        for _ in range(4):
            for w in ws:
                proj.floatMatvec(x, out, w, n, d)
            ctx.sync()
        shapes["gemv %s %d x %d" % (name, d, n)] = int(host.size)
        for w in ws:
            w.free()
    for name, d, n in (("Q4_K", 4096, 12288), ("Q4_K", 4096, 11008), ("Q8_0", 4096, 11008), ("Q4_K", 3584, 18944)):
        t = GGMLType[name]
        host = synthetic.weight(t, d, n, 97)
        ws = [ctx.load_weight(t, host, d, n) for _ in range(3)]
        for B in (8, 64, 96):
            X, out = ctx.from_numpy(synthetic.activations((B, n), 98 + B)), ctx.float_array(B * d)
            proj = QuantizedBatchProjections(ctx, B, n, d)
            for _ in range(4):
                for w in ws:
                    proj.projection(X, out, w, n, d, True)
                ctx.sync()
            proj.workspace.free()
        shapes["batched %s %d x %d" % (name, d, n)] = int(host.size)
        for w in ws:
            w.free()
    print(json.dumps({"weight_bytes": shapes}))


def int8_probe(ctx, t, T=2048):
    """What the counters and the kernel trace of the int8 prefill path are collected on: one
    Llama-3.2-1B layer's four calls at T tokens with JL_MATH_INT8, kernel by kernel, four times."""
    from jitllm_amd import _lib as L, synthetic
    from jitllm_amd.projections import QuantizedBatchProjections
    shapes = {"wq": (DIM, DIM), "wk": (KV_DIM, DIM), "wv": (KV_DIM, DIM), "wo": (DIM, DIM),
              "w1": (HIDDEN, DIM), "w3": (HIDDEN, DIM), "w2": (DIM, HIDDEN)}
    w = {k: ctx.load_weight(t, synthetic.weight(t, r, c, 41 + i), r, c) for i, (k, (r, c)) in enumerate(shapes.items())}
    X = ctx.from_numpy(synthetic.activations((T, DIM), 48))
    H = ctx.from_numpy(synthetic.activations((T, HIDDEN), 49) * np.float32(0.1))
    qkv, res, hb = ctx.float_array(T * (DIM + 2 * KV_DIM)), ctx.float_array(T * DIM, fill=0.0), ctx.float_array(T * HIDDEN)
    proj = QuantizedBatchProjections(ctx, T, HIDDEN, 2 * HIDDEN, math=L.JL_MATH_INT8)
    for _ in range(4):
        proj.fusedQKV(X, qkv, w["wq"], w["wk"], w["wv"])
        proj.projection(X, res, w["wo"], DIM, DIM, True)
        proj.gateUp(X, hb, w["w1"], w["w3"], DIM, HIDDEN)
        proj.projection(H, res, w["w2"], HIDDEN, DIM, True)
        ctx.sync()
    print(json.dumps({"tokens": T, "macs": {"q|k|v": T * DIM * (DIM + 2 * KV_DIM), "o": T * DIM * DIM,
                                            "gate/up": T * 2 * HIDDEN * DIM, "down": T * HIDDEN * DIM}}))


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline legs")
    ap.add_argument("--no-extra", action="store_true", help="skip the legs beside the decode set")
    ap.add_argument("--extra", default="wq_shape,fused_rms,prefill,other_types,batched,prefill_other_types,batched_other_types,batched_vocabulary,short_prompt",
                    help="comma-separated legs beside the decode set (a profiler run takes a few at a time)")
    ap.add_argument("--prefill-warmup", type=int, default=-1,
                    help="untimed replays before the prefill legs (default 100; 10 under a profiler)")
    ap.add_argument("--traffic-probe", action="store_true",
                    help="only launch what the HBM-traffic counters are read on (see traffic_probe)")
    ap.add_argument("--prefill-probe", action="store_true",
                    help="only launch what the matrix-pipe counters are read on (see prefill_probe)")
    ap.add_argument("--probe-tokens", type=int, default=2048, help="--prefill-probe: tokens")
    ap.add_argument("--probe-mode", default="xf16", choices=["xf16", "resident", "default"],
                    help="--prefill-probe: operand types and residency (see prefill_probe)")
    ap.add_argument("--hbm-rate-probe", action="store_true",
                    help="only measure the rate of a plain streaming read of HBM (see hbm_rate_probe)")
    ap.add_argument("--mfma-rate-probe", action="store_true",
                    help="only measure the sustained rate of fp16 matrix instructions (see mfma_rate_probe)")
    ap.add_argument("--vocabulary-probe", action="store_true",
                    help="only launch the batched vocabulary projection and its per-row argmax (see vocabulary_probe)")
    ap.add_argument("--shapes-probe", action="store_true",
                    help="long single-token rows and awkward batched row lengths, kernel by kernel (for rocprofv3)")
    ap.add_argument("--batched-probe", action="store_true",
                    help="only launch the batched-decode calls, kernel by kernel (see batched_probe)")
    ap.add_argument("--decode-probe", action="store_true",
                    help="only launch the decode kernels, kernel by kernel (see decode_probe)")
    ap.add_argument("--roofline-probe", action="store_true",
                    help="only replay the roofline leg's graph of gate/up launches (see roofline_probe)")
    ap.add_argument("--int8-probe", action="store_true",
                    help="only launch the int8 prefill calls, kernel by kernel (see int8_probe)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: the path is built and measured on a single MI355X; "
              "run with --gpus 1", file=sys.stderr)
        sys.exit(2)

    from jitllm_amd.ggml import GGMLType
    from jitllm_amd.projections import QuantizedProjections, TornadoWorkspace
    from jitllm_amd.runtime import Context

    t = GGMLType.Q8_0
    hip = Hip()
    cpu = not args.no_cpu
    # (the matrix pipe's clock takes tens of milliseconds of load to settle: 100 untimed replays of
    # the layer before the timed ones; a kernel tracer records every one of them, so few then)
    prefill_warmup = args.prefill_warmup if args.prefill_warmup >= 0 else (10 if under_tracer() else 100)
    with Context(0) as ctx:
        cu, name = ctx.device_info()
        clock_khz = hip.clock_khz(0)
        if args.mfma_rate_probe:
            print(json.dumps(mfma_rate_probe(cu)))
            return
        if args.hbm_rate_probe:
            print(json.dumps(hbm_rate_probe(cu)))
            return
        if args.prefill_probe:
            prefill_probe(ctx, t, args.probe_tokens, args.probe_mode)
            return
        if args.vocabulary_probe:
            vocabulary_probe(ctx)
            return
        if args.batched_probe:
            batched_probe(ctx)
            return
        if args.shapes_probe:
            shapes_probe(ctx)
            return
        if args.int8_probe:
            int8_probe(ctx, t)
            return
        layers, wcls, acts, host, shapes = build_decode_set(ctx, t)
        ws = TornadoWorkspace(wrapX=acts["x"], wrapXb=acts["xb"], wrapHb=acts["hb"])
        proj = QuantizedProjections(ctx, ws)
        if args.traffic_probe:
            traffic_probe(ctx, proj, layers)
            return
        if args.decode_probe:
            decode_probe(ctx, proj, layers, wcls, acts)
            return
        if args.roofline_probe:
            roofline_probe(ctx, hip, proj, layers)
            return
        total_bytes = decode_bytes()
        assert total_bytes == 1316320256, total_bytes

        # result check, before anything is timed: the gate/up launch and the vocabulary projection
        x0, xb0 = acts["x"].get(), acts["xb"].get()
        proj.gateUp(layers[-1]["w1"], layers[-1]["w3"], DIM, HIDDEN)
        proj.floatMatvec(acts["xb"], acts["logits"], wcls, DIM, VOCAB)
        proj.fusedQKV(acts["xb"], acts["q"], acts["k"], acts["v"], layers[0]["wq"], layers[0]["wk"], layers[0]["wv"])
        proj.residualMatvec(acts["xb"], layers[0]["wo"], DIM, DIM)
        ctx.sync()
        checks = {}
        rh, rv, rd = sample_rows(HIDDEN, 96, 1), sample_rows(VOCAB, 160, 2), sample_rows(DIM, 96, 3)
        g, mg = oracle_rows(t, host["w1"], DIM, rh, xb0)
        u, mu = oracle_rows(t, host["w3"], DIM, rh, xb0)
        checks["gate/up"] = check_swiglu("decode gate/up", acts["hb"].get()[rh], g[0], u[0], mg[0], mu[0], 1e-3)
        ref, mag = oracle_rows(t, host["wcls"], DIM, rv, xb0)
        checks["vocabulary"] = check("vocabulary projection", acts["logits"].get()[rv], ref[0], mag[0], 1e-3)
        ref, mag = oracle_rows(t, host["wq"], DIM, rd, xb0)
        checks["q"] = check("decode q", acts["q"].get()[rd], ref[0], mag[0], 1e-3)
        ref, mag = oracle_rows(t, host["wo"], DIM, rd, xb0)
        checks["o (residual)"] = check("decode o", acts["x"].get()[rd] - x0[rd].astype(np.float64), ref[0],
                                       mag[0] + np.abs(x0[rd]) * 1e-6, 1e-3)

        for _ in range(max(1, args.warmup)):
            decode_step(proj, layers, wcls, acts)
        ctx.sync()

        # A step is replayed as a HIP graph of its 65 launches: Python cannot enqueue a kernel in
        # less than a few microseconds, which is longer than several of these kernels run.
        stream = ctx.stream
        step_graph = hip.capture(stream, lambda: decode_step(proj, layers, wcls, acts))
        for _ in range(args.warmup):
            hip.launch(step_graph, stream)
        ctx.sync()

        # timed region: REPS repetitions of exactly K steps each; the median repetition is reported
        step_ms, walls = [], []
        for _ in range(REPS):
            e0, e1 = hip.event(), hip.event()
            ctx.sync()
            t0 = time.perf_counter()
            hip.record(e0, stream)
            for _ in range(args.steps):
                hip.launch(step_graph, stream)
            hip.record(e1, stream)
            ctx.sync()
            walls.append((time.perf_counter() - t0) * 1e3 / args.steps)
            step_ms.append(hip.elapsed_ms(e0, e1) / args.steps)
            hip.destroy_event(e0)
            hip.destroy_event(e1)
        hip.destroy_graph(step_graph)
        ms = statistics.median(step_ms)

        # the same K steps launched kernel by kernel from Python, for comparison (never the headline)
        e0, e1 = hip.event(), hip.event()
        hip.record(e0, stream)
        for _ in range(args.steps):
            decode_step(proj, layers, wcls, acts)
        hip.record(e1, stream)
        ms_python = hip.elapsed_ms(e0, e1) / args.steps
        hip.destroy_event(e0)
        hip.destroy_event(e1)

        # the step's kernels on their own, each as a graph over the 16 layers' own weights (so
        # nothing is served from the 256 MB memory-side cache)
        # (four sweeps of the layers to a graph: the ~7 us pause that follows every replay is then
        # shared by 64 launches and is not what a launch is charged)
        def per_kernel(fn, launches, nbytes):
            def sweeps():
                for _ in range(4):
                    fn()
            us = [m / (4 * launches) * 1e3 for m in timed_graph(ctx, hip, sweeps, max(4, args.steps // 4), 2)]
            med = statistics.median(us)
            return {"avg_launch_us": round(med, 3), "us_stats": spread_stats(us, 1.0, 3),
                    "bytes_per_launch": nbytes, "GB_s": round(nbytes / med / 1e3, 1),
                    "frac_hbm_peak": round(nbytes / med / 1e3 / HBM_PEAK_GBS, 4)}

        def gate_ups():
            for w in layers:
                proj.gateUp(w["w1"], w["w3"], DIM, HIDDEN)

        def qkvs():
            for w in layers:
                proj.fusedQKV(acts["xb"], acts["q"], acts["k"], acts["v"], w["wq"], w["wk"], w["wv"])

        def os_():
            for w in layers:
                proj.residualMatvec(acts["xb"], w["wo"], DIM, DIM)

        def downs():
            for w in layers:
                proj.residualMatvec(acts["hb"], w["w2"], HIDDEN, DIM)
        gate_up_bytes = 2 * gemv_bytes(HIDDEN, DIM)
        gu = per_kernel(gate_ups, LAYERS, gate_up_bytes)
        kernels = {
            "gate/up 2 x [8192 x 2048]": gu,
            "q|k|v [3072 x 2048]": per_kernel(qkvs, LAYERS, gemv_bytes(DIM, DIM) + 2 * gemv_bytes(KV_DIM, DIM)),
            "o [2048 x 2048] +=": per_kernel(os_, LAYERS, gemv_bytes(DIM, DIM)),
            "down [2048 x 8192] +=": per_kernel(downs, LAYERS, gemv_bytes(DIM, HIDDEN)),
        }
        # the vocabulary projection over two device copies of its weight in turn (2 x 280 MB: what
        # one launch reads, the memory-side cache has lost by the time the launch comes round again)
        wcls_b = ctx.load_weight(t, host["wcls"], VOCAB, DIM)

        def vocabs():
            for w in (wcls, wcls_b):
                proj.floatMatvec(acts["xb"], acts["logits"], w, DIM, VOCAB)
        kernels["vocabulary [128256 x 2048]"] = per_kernel(vocabs, 2, gemv_bytes(VOCAB, DIM))
        wcls_b.free()
        # the single-weight instances of the tile kernel (q|k|v, o, down, vocabulary) together:
        # everything in the step that is not a gate/up launch
        single_bytes = total_bytes - LAYERS * gate_up_bytes
        single_ms = ms - LAYERS * gu["avg_launch_us"] * 1e-3
        gbs = total_bytes / (ms * 1e-3) / 1e9
        achieved = gu["GB_s"]
        out = {
            "metric": "Q-GEMV HBM GB/s (% of peak) + prefill tok/s (% MFMA peak), 1xMI355X",
            "value": round(gbs, 1), "unit": "GB/s", "n_gpus": 1, "steps": args.steps,
            "warmup": args.warmup, "ms_per_step": round(ms, 4), "higher_is_better": True,
            "scaling": "weak", "vs_baseline": None, "dtype": "f32",
            "data": "synthetic (seeded Q8_0 blocks; one layer's host bytes uploaded into 16 distinct "
                    "device buffers)",
            "config": {"workload": "Q8_0 Llama-3.2-1B decode projection set, batch 1: 16 x (q|k|v, o, "
                                   "gate/up SwiGLU, down) + vocabulary projection, 65 launches/token "
                                   "replayed as one HIP graph",
                       "bytes_per_step": total_bytes, "device": name, "compute_units": cu,
                       "peak_clock_khz": clock_khz},
            "frac_hbm_peak": round(gbs / HBM_PEAK_GBS, 4),
            "tok_s": round(1e3 / ms, 1),
            "ms_per_step_stats": spread_stats(step_ms),
            "ms_per_step_python_launches": round(ms_python, 4),
            "host_wall_ms_per_step": round(statistics.median(walls), 4),
            "checks_rel_err": checks,
            "roofline": {"bound": "hbm",
                         "kernel": "jl_gemv_tiles<Q8_0, gate/up> 2 x [8192 x 2048]: the largest launch "
                                   "shape of the step (16 of its 65 launches, 43 % of its bytes), not its "
                                   "slowest -- see step_frac and single_weight_launches",
                         "achieved": achieved, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                         "frac": round(achieved / HBM_PEAK_GBS, 4), "traffic": GATE_UP_HBM_TRAFFIC_BYTES,
                         "bytes_per_launch": gate_up_bytes,
                         "avg_launch_us": gu["avg_launch_us"], "launch_us_stats": gu["us_stats"],
                         "launches_timed": max(4, args.steps // 4) * 4 * LAYERS * REPS,
                         "step_frac": round(gbs / HBM_PEAK_GBS, 4),
                         "single_weight_launches": {
                             "what": "the 49 launches of a step that are not gate/up (q|k|v, o, down, vocabulary)",
                             "bytes": single_bytes, "ms": round(single_ms, 4),
                             "GB_s": round(single_bytes / (single_ms * 1e-3) / 1e9, 1),
                             "frac": round(single_bytes / (single_ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4)}},
            "decode_kernels": kernels,
        }
        # what a plain read loop streams from HBM on this box, beside the published peak
        hbm = hbm_rate_probe(cu)
        out["roofline"]["sustained_from_box"] = dict(
            hbm, frac_of_sustained=round(achieved / hbm["hbm_read_GB_s"], 4),
            step_frac_of_sustained=round(gbs / hbm["hbm_read_GB_s"], 4))
        legs = set() if args.no_extra else set(args.extra.split(","))
        if "wq_shape" in legs:
            out["wq_shape"] = bench_wq_shape(ctx, hip, t, args.steps, args.warmup, cpu)
        if "fused_rms" in legs:
            out["decode_fused_rms"] = bench_fused_rms(ctx, hip, proj, layers, wcls, acts, host, args.steps,
                                                      args.warmup)
        if "prefill" in legs:
            out["prefill"] = [bench_gemm(ctx, hip, t, T, max(4, args.steps // 2), prefill_warmup, cpu and T == 512,
                                         clock_khz, cu) for T in (512, 2048)]
            # what the matrix pipe sustains on this box, beside the published peak the fractions use
            sustained = mfma_rate_probe(cu)
            for leg in out["prefill"]:
                leg["roofline"]["sustained_from_box"] = dict(
                    sustained, frac_of_random_operand_rate=round(
                        leg["roofline"]["achieved"] / sustained["16x16x32_random_operands"], 4))
        if "other_types" in legs:
            out["decode_other_types"] = [
                bench_decode_layers(ctx, hip, "Q4_0", 4096, 1024, 14336, OTHER_TYPE_COPIES, args.steps, args.warmup, cpu),
                bench_decode_layers(ctx, hip, "Q4_K", 4096, 1024, 12288, OTHER_TYPE_COPIES, args.steps, args.warmup, cpu)]
        if "batched" in legs:
            out["batched_q4k"] = [bench_batched(ctx, hip, B, max(5, args.steps // 5), 3, cpu)
                                  for B in (8, 32, 64)]
        if "prefill_other_types" in legs:
            # the prefill GEMM of the other two weight types at 8B-model shapes: Q4_K is decoded to
            # fp16 (in LDS or once per call) and multiplied on the fp16 MFMA, Q4_0 likewise by default
            out["prefill_other_types"] = [
                bench_gemm(ctx, hip, GGMLType[name], T, max(4, args.steps // 4), prefill_warmup // 2, cpu and T == 512,
                           clock_khz, cu, dims=dims, int8=False, model=model)
                for name, dims, model in (("Q4_K", (4096, 1024, 12288), "Qwen3-8B-like"),
                                          ("Q4_0", (4096, 1024, 14336), "Llama-3-8B"))
                for T in (512, 2048)]
        if "batched_other_types" in legs:
            # batched decode of the other two weight types: Q8_0 at Llama-3.2-1B shapes (32 layer
            # copies of 65 MB to a replay), Q4_0 at Llama-3-8B shapes
            out["batched_other_types"] = [
                bench_batched(ctx, hip, B, max(5, args.steps // 5), 3, cpu, name, dims, model, copies)
                for name, dims, model, copies in (("Q8_0", (DIM, KV_DIM, HIDDEN), "Llama-3.2-1B", 32),
                                                  ("Q4_0", (4096, 1024, 14336), "Llama-3-8B", 8))
                for B in (8, 32, 64)]
        if "batched_vocabulary" in legs:
            # the other launch of a batched decode step: logits for B sequences
            out["batched_vocabulary"] = [
                bench_batched_vocabulary(ctx, hip, name, vocab, dim, model, (8, 32, 64), max(10, args.steps // 2), 3)
                for name, vocab, dim, model in (("Q4_K", 151936, 4096, "Qwen3-8B-like"), ("Q8_0", VOCAB, DIM, "Llama-3.2-1B"))]
        if "short_prompt" in legs:
            # between batched decode and prefill: 96, 192 and 384 rows (most prompts are this long)
            out["short_prompt"] = bench_short_prompt(ctx, hip, (96, 192, 384), max(5, args.steps // 5), 3)
        out["cpu_baseline"] = cpu_baseline(host, shapes, t) if cpu else None
    print(json.dumps(out))


if __name__ == "__main__":
    main()
