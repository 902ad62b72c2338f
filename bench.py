#!/usr/bin/env python3
"""Benchmark of the quantized weight-matmul hot path on one MI355X.

A step is one pass of the decode projection set of Llama-3.2-1B in Q8_0, batch 1 -- per layer the
fused q|k|v projection, the output projection (residual), the fused gate/up SwiGLU projection and
the down projection (residual), 16 layers, then the 2048 -> 128256 vocabulary projection: 65 kernel
launches, 1 316 320 256 algorithmic bytes (weights in GGUF block layout + fp32 input + fp32 output,
each once).  Inputs are resident in HBM before the timed region.  Every layer owns distinct device
buffers, so the 1.3 GB sweep cannot live in the 256 MB memory-side cache.

Prints one JSON line.  `value` is GB/s of algorithmic bytes; `roofline` is the dominant kernel
(the fused gate/up GEMV) against the 8 TB/s HBM peak; `cpu_baseline` is the oracle's restatement of
the reference's Java CPU matmul timed on this machine's host cores; `prefill` and `batched` carry
the MFMA side of the metric.
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

# Llama-3.2-1B geometry: the decode projection set the headline metric is quoted on
DIM, KV_DIM, HIDDEN, VOCAB, LAYERS = 2048, 512, 8192, 128256, 16


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


def decode_step_fused_rms(proj, layers, wcls, acts):
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
    proj.rmsMatvec(acts["x"], acts["rms_final"], None, acts["logits"], wcls, DIM, VOCAB, eps=1e-5)
    proj.argmax(acts["logits"], VOCAB, acts["token"])


def bench_fused_rms(ctx, hip, proj, layers, wcls, acts, steps, warmup):
    from jitllm_amd import synthetic
    for i, k in enumerate(("rms_att", "rms_ffn", "rms_final")):
        acts[k] = ctx.from_numpy((1.0 + 0.1 * synthetic.activations(DIM, 31 + i)).astype("float32"))
    acts["token"] = ctx.raw_buffer(4)
    stream = ctx.stream
    decode_step_fused_rms(proj, layers, wcls, acts)
    ctx.sync()
    graph = hip.capture(stream, lambda: decode_step_fused_rms(proj, layers, wcls, acts))
    for _ in range(warmup):
        hip.launch(graph, stream)
    e0, e1 = hip.event(), hip.event()
    hip.record(e0, stream)
    for _ in range(steps):
        hip.launch(graph, stream)
    hip.record(e1, stream)
    ctx.sync()
    ms = hip.elapsed_ms(e0, e1) / steps
    return {"ms_per_step": round(ms, 4), "tok_s": round(1e3 / ms, 1), "launches": 4 * LAYERS + 2,
            "what": "decode set with the 33 RMS normalisations folded into q|k|v, gate/up and the "
                    "vocabulary projection (scale computed inside each kernel, no normalised vector "
                    "written) and the greedy token chosen on the device"}


def decode_bytes():
    """Algorithmic bytes of a step: every one of the 7 projections of a layer counted on its own
    (weight blocks + fp32 input + fp32 output), as the benchmark's definition does, even where one
    launch serves several of them."""
    per_layer = (gemv_bytes(DIM, DIM) + 2 * gemv_bytes(KV_DIM, DIM) + gemv_bytes(DIM, DIM)
                 + 2 * gemv_bytes(HIDDEN, DIM) + gemv_bytes(DIM, HIDDEN))
    return LAYERS * per_layer + gemv_bytes(VOCAB, DIM)


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
    times = []
    begin = time.perf_counter()
    while len(times) < 4 or (time.perf_counter() - begin < budget_s and len(times) < 5000):
        t0 = time.perf_counter()
        for k in names:
            rows, cols = shapes[k]
            O.matmul(int(t), host[k], x_hid if cols == HIDDEN else x_dim, rows, cols,
                     O.DOT_VEC256, threads)
        times.append(time.perf_counter() - t0)
    med = statistics.median(times[1:])
    return {"value": round(nbytes / med / 1e9, 2), "unit": "GB/s", "cores": threads, "kind": "port",
            "sample": f"one layer's 7 projections + vocabulary projection ({nbytes} B), "
                      f"median of {len(times) - 1} passes after 1 warm-up "
                      f"({time.perf_counter() - begin:.1f} s of wall time), 256-bit vectorDot order",
            "tok_s_equiv": round(nbytes / med / decode_bytes(), 3)}


def bench_gemm(ctx, hip, t, T, steps, warmup):
    """Batched prefill of one Llama-3.2-1B layer (q|k|v, o, gate/up SwiGLU, down) over T tokens."""
    from jitllm_amd import synthetic
    from jitllm_amd.projections import QuantizedBatchProjections
    w = {
        "wq": ctx.load_weight(t, synthetic.weight(t, DIM, DIM, 41), DIM, DIM),
        "wk": ctx.load_weight(t, synthetic.weight(t, KV_DIM, DIM, 42), KV_DIM, DIM),
        "wv": ctx.load_weight(t, synthetic.weight(t, KV_DIM, DIM, 43), KV_DIM, DIM),
        "wo": ctx.load_weight(t, synthetic.weight(t, DIM, DIM, 44), DIM, DIM),
        "w1": ctx.load_weight(t, synthetic.weight(t, HIDDEN, DIM, 45), HIDDEN, DIM),
        "w3": ctx.load_weight(t, synthetic.weight(t, HIDDEN, DIM, 46), HIDDEN, DIM),
        "w2": ctx.load_weight(t, synthetic.weight(t, DIM, HIDDEN, 47), DIM, HIDDEN),
    }
    X = ctx.from_numpy(synthetic.activations((T, DIM), 48))
    H = ctx.from_numpy(synthetic.activations((T, HIDDEN), 49) * np.float32(0.1))
    qkv = ctx.float_array(T * (DIM + 2 * KV_DIM))
    res = ctx.float_array(T * DIM, fill=0.0)
    hb = ctx.float_array(T * HIDDEN)
    X16 = ctx.half_from_numpy(synthetic.activations((T, DIM), 48))
    H16 = ctx.half_from_numpy(synthetic.activations((T, HIDDEN), 49) * np.float32(0.1))
    hb16 = ctx.half_array(T * HIDDEN)
    def timed(proj, X=X, H=H, hb=hb):
        def layer():
            proj.fusedQKV(X, qkv, w["wq"], w["wk"], w["wv"])
            proj.projection(X, res, w["wo"], DIM, DIM, True)
            proj.gateUp(X, hb, w["w1"], w["w3"], DIM, HIDDEN)
            proj.projection(H, res, w["w2"], HIDDEN, DIM, True)

        # replayed as a HIP graph: Python cannot enqueue the layer's launches as fast as they run
        layer()
        ctx.sync()
        graph = hip.capture(ctx.stream, layer)
        for _ in range(warmup):
            hip.launch(graph, ctx.stream)
        ctx.sync()
        e0, e1 = hip.event(), hip.event()
        hip.record(e0, ctx.stream)
        for _ in range(steps):
            hip.launch(graph, ctx.stream)
        hip.record(e1, ctx.stream)
        return hip.elapsed_ms(e0, e1) / steps

    ms = timed(QuantizedBatchProjections(ctx, T, HIDDEN, 2 * HIDDEN))
    # the reference's residency choice: an fp16 copy per projection kept across calls (2 bytes per
    # weight of HBM), decoded by the first call only -- reported beside the default, not instead
    ms_kept = timed(QuantizedBatchProjections(ctx, T, HIDDEN, 2 * HIDDEN, resident=True))
    # the reference's own operand types on top of that: activations arrive as fp16 (its RMS apply,
    # attention and SwiGLU kernels write fp16) and the hidden vector leaves as fp16
    ms_half = timed(QuantizedBatchProjections(ctx, T, HIDDEN, 2 * HIDDEN, resident=True), X16, H16, hb16)
    # what hands the projections those fp16 rows: the RMS reduction and fp16 apply of one [T x dim]
    # activation (two per layer in the model), timed on its own
    rms_w = ctx.from_numpy(np.ones(DIM, dtype=np.float32))
    half_proj = QuantizedBatchProjections(ctx, T, DIM, DIM)
    def rms_apply():
        # (8 launches per graph: a one-kernel graph measures the graph launch, not the kernel)
        for _ in range(8):
            half_proj.rmsApplyFP16(X, rms_w, 1e-5, X16, DIM)
    rms_apply()
    ctx.sync()
    graph = hip.capture(ctx.stream, rms_apply)
    for _ in range(3):
        hip.launch(graph, ctx.stream)
    ctx.sync()
    e0, e1 = hip.event(), hip.event()
    hip.record(e0, ctx.stream)
    for _ in range(steps):
        hip.launch(graph, ctx.stream)
    hip.record(e1, ctx.stream)
    rms_us = hip.elapsed_ms(e0, e1) / steps / 8 * 1e3
    flops = 2.0 * T * (DIM * (DIM + 2 * KV_DIM) + DIM * DIM + 2 * DIM * HIDDEN + HIDDEN * DIM)
    tflops = flops / (ms * 1e-3) / 1e12
    tflops_kept = flops / (ms_kept * 1e-3) / 1e12
    tflops_half = flops / (ms_half * 1e-3) / 1e12
    return {"tokens": T, "ms_per_layer": round(ms, 4), "tok_s_16_layers": round(T / (ms * 1e-3 * LAYERS), 1),
            "tflops": round(tflops, 1), "frac_f16_mfma_peak": round(tflops / F16_MFMA_PEAK_TFLOPS, 4),
            "math": "f16 MFMA, fp32 accumulate; weights decoded to fp16 inside the call (in LDS, or once per call into the workspace)",
            "with_resident_fp16_copy": {"ms_per_layer": round(ms_kept, 4), "tflops": round(tflops_kept, 1),
                                        "frac_f16_mfma_peak": round(tflops_kept / F16_MFMA_PEAK_TFLOPS, 4)},
            "with_resident_copy_and_fp16_activations": {
                "ms_per_layer": round(ms_half, 4), "tflops": round(tflops_half, 1),
                "frac_f16_mfma_peak": round(tflops_half / F16_MFMA_PEAK_TFLOPS, 4),
                "rms_apply_to_fp16_us": round(rms_us, 2)}}


def bench_batched_q4k(ctx, hip, B, steps, warmup):
    """Q4_K batched decode, Qwen3-8B-like shapes (dim 4096, ffn 12288, kv 1024), B sequences."""
    from jitllm_amd import synthetic
    from jitllm_amd.ggml import GGMLType
    from jitllm_amd.projections import QuantizedBatchProjections
    t = GGMLType.Q4_K
    dim, kv, ffn = 4096, 1024, 12288
    w = {
        "wq": ctx.load_weight(t, synthetic.weight(t, dim, dim, 61), dim, dim),
        "wk": ctx.load_weight(t, synthetic.weight(t, kv, dim, 62), kv, dim),
        "wv": ctx.load_weight(t, synthetic.weight(t, kv, dim, 63), kv, dim),
        "wo": ctx.load_weight(t, synthetic.weight(t, dim, dim, 64), dim, dim),
        "w1": ctx.load_weight(t, synthetic.weight(t, ffn, dim, 65), ffn, dim),
        "w3": ctx.load_weight(t, synthetic.weight(t, ffn, dim, 66), ffn, dim),
        "w2": ctx.load_weight(t, synthetic.weight(t, dim, ffn, 67), dim, ffn),
    }
    X = ctx.from_numpy(synthetic.activations((B, dim), 68))
    H = ctx.from_numpy(synthetic.activations((B, ffn), 69) * np.float32(0.1))
    qkv = ctx.float_array(B * (dim + 2 * kv))
    res = ctx.float_array(B * dim, fill=0.0)
    hb = ctx.float_array(B * ffn)
    proj = QuantizedBatchProjections(ctx, B, ffn, 2 * ffn)

    def layer():
        proj.fusedQKV(X, qkv, w["wq"], w["wk"], w["wv"])
        proj.projection(X, res, w["wo"], dim, dim, True)
        proj.gateUp(X, hb, w["w1"], w["w3"], dim, ffn)
        proj.projection(H, res, w["w2"], ffn, dim, True)

    # replayed as a HIP graph: Python cannot enqueue the layer's launches as fast as they run
    layer()
    ctx.sync()
    graph = hip.capture(ctx.stream, layer)
    for _ in range(warmup):
        hip.launch(graph, ctx.stream)
    ctx.sync()
    e0, e1 = hip.event(), hip.event()
    hip.record(e0, ctx.stream)
    for _ in range(steps):
        hip.launch(graph, ctx.stream)
    hip.record(e1, ctx.stream)
    ms = hip.elapsed_ms(e0, e1) / steps
    wbytes = sum(x.nbytes for x in w.values())
    # fp32 activations in and out, once per projection
    io = 4 * B * (dim + dim + 2 * kv + dim + dim + dim + ffn + ffn + dim)
    flops = 2.0 * B * (dim * (dim + 2 * kv) + dim * dim + 2 * dim * ffn + ffn * dim)
    gbs = (wbytes + io) / (ms * 1e-3) / 1e9
    return {"B": B, "ms_per_layer": round(ms, 4), "GB_s": round(gbs, 1),
            "frac_hbm_peak": round(gbs / HBM_PEAK_GBS, 4),
            "tflops": round(flops / (ms * 1e-3) / 1e12, 1), "bytes": wbytes + io}


def bench_decode_layers(ctx, hip, type_name, dim, kv, ffn, copies, steps, warmup):
    """Single-token decode projections of one layer -- q|k|v, o (+=), gate/up SwiGLU, down (+=) --
    over `copies` distinct layers' weights (more bytes than the 256 MB last-level cache holds),
    replayed as one HIP graph.  Q4_0 at Llama-3-8B shapes and Q4_K at Qwen3-8B-like shapes: the
    other two weight types the path is specified on.  Timed twice: the fp32-activation path (the one
    held to the CPU path's results) and the reference's optional packed-integer path, whose four
    activation quantisations per layer are launches of their own here and are counted."""
    from jitllm_amd import synthetic
    from jitllm_amd.ggml import GGMLType
    from jitllm_amd.projections import PackedActivation, QuantizedProjections, TornadoWorkspace
    t = GGMLType[type_name]
    shapes = {"wq": (dim, dim), "wk": (kv, dim), "wv": (kv, dim), "wo": (dim, dim),
              "w1": (ffn, dim), "w3": (ffn, dim), "w2": (dim, ffn)}
    host = {k: synthetic.weight(t, r, c, 71 + i) for i, (k, (r, c)) in enumerate(shapes.items())}
    layers = [{k: ctx.load_weight(t, host[k], *shapes[k]) for k in shapes} for _ in range(copies)]
    x = ctx.from_numpy(synthetic.activations(dim, 78))
    xb = ctx.from_numpy(synthetic.activations(dim, 79))
    q, k_, v = ctx.float_array(dim), ctx.float_array(kv), ctx.float_array(kv)
    hb = ctx.from_numpy(synthetic.activations(ffn, 80) * np.float32(0.1))
    hb2 = ctx.float_array(ffn)
    proj = QuantizedProjections(ctx, TornadoWorkspace(wrapX=x, wrapXb=xb, wrapHb=hb2, wrapHb2=hb))
    small = QuantizedProjections(ctx, TornadoWorkspace(wrapHb=hb2, packedX=PackedActivation(ctx, dim)), packed=True)
    wide = QuantizedProjections(ctx, TornadoWorkspace(packedX=PackedActivation(ctx, ffn)), packed=True)

    def step():
        for w in layers:
            proj.fusedQKV(xb, q, k_, v, w["wq"], w["wk"], w["wv"])
            proj.residualMatvec(xb, w["wo"], dim, dim)
            proj.gateUp(w["w1"], w["w3"], dim, ffn)
            proj.residualMatvec(hb, w["w2"], ffn, dim)

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

    def timed(fn):
        fn()
        ctx.sync()
        graph = hip.capture(ctx.stream, fn)
        for _ in range(warmup):
            hip.launch(graph, ctx.stream)
        ctx.sync()
        e0, e1 = hip.event(), hip.event()
        hip.record(e0, ctx.stream)
        for _ in range(steps):
            hip.launch(graph, ctx.stream)
        hip.record(e1, ctx.stream)
        return hip.elapsed_ms(e0, e1) / steps / copies

    ms = timed(step)
    ms_packed = timed(step_packed)
    wbytes = sum(a.size for a in host.values())
    io = 4 * (dim + dim + 2 * kv + dim + dim + dim + ffn + ffn + dim)
    gbs = (wbytes + io) / (ms * 1e-3) / 1e9
    return {"type": type_name, "shapes": {"dim": dim, "kv": kv, "ffn": ffn}, "layers_swept": copies,
            "ms_per_layer": round(ms, 4), "GB_s": round(gbs, 1), "frac_hbm_peak": round(gbs / HBM_PEAK_GBS, 4),
            "bytes_per_layer": wbytes + io,
            "packed_activation_path": {"ms_per_layer": round(ms_packed, 4), "launches_per_layer": 8,
                                       "GB_s": round((wbytes + io) / (ms_packed * 1e-3) / 1e9, 1)}}


# HBM bytes one gate/up launch moves, from `rocprofv3 --pmc FETCH_SIZE` and `--pmc WRITE_SIZE` over
# `bench.py --traffic-probe` (profiles/gemv_q8_0_gate_up_hbm_traffic.md): 17 517 KiB x 2.0 read
# (the counter books 64 bytes for each of this chip's 128-byte requests; a 256 MiB plain copy reads
# 131 088 KiB on it) + 64 KiB x 1.0 written.  The algorithmic figure is 35 733 504 bytes.
GATE_UP_HBM_TRAFFIC_BYTES = 17517 * 1024 * 2 + 64 * 1024


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


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-extra", action="store_true", help="skip the prefill / batched legs")
    ap.add_argument("--extra", default="fused_rms,prefill,other_types,batched",
                    help="comma-separated legs beside the decode set (a profiler run takes a few at a time)")
    ap.add_argument("--traffic-probe", action="store_true",
                    help="only launch what the HBM-traffic counters are read on (see traffic_probe)")
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
    with Context(0) as ctx:
        cu, name = ctx.device_info()
        layers, wcls, acts, host, shapes = build_decode_set(ctx, t)
        ws = TornadoWorkspace(wrapX=acts["x"], wrapXb=acts["xb"], wrapHb=acts["hb"])
        proj = QuantizedProjections(ctx, ws)
        if args.traffic_probe:
            traffic_probe(ctx, proj, layers)
            return
        total_bytes = decode_bytes()
        assert total_bytes == 1316320256, total_bytes

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

        # timed region: exactly K steps
        e0, e1 = hip.event(), hip.event()
        t0 = time.perf_counter()
        hip.record(e0, stream)
        for _ in range(args.steps):
            hip.launch(step_graph, stream)
        hip.record(e1, stream)
        ctx.sync()
        wall = time.perf_counter() - t0
        ms_step_clean = hip.elapsed_ms(e0, e1) / args.steps

        # the same K steps launched kernel by kernel from Python, for comparison
        hip.record(e0, stream)
        for _ in range(args.steps):
            decode_step(proj, layers, wcls, acts)
        hip.record(e1, stream)
        ms_step = hip.elapsed_ms(e0, e1) / args.steps

        # dominant kernel: the fused gate/up GEMV, 16 launches over the 16 layers' own weights
        # (571 MB, so nothing is served from the 256 MB memory-side cache), replayed K times
        def gate_ups():
            for w in layers:
                proj.gateUp(w["w1"], w["w3"], DIM, HIDDEN)
        gu_graph = hip.capture(stream, gate_ups)
        hip.launch(gu_graph, stream)
        hip.record(e0, stream)
        for _ in range(args.steps):
            hip.launch(gu_graph, stream)
        hip.record(e1, stream)
        gate_up_avg = hip.elapsed_ms(e0, e1) / (args.steps * LAYERS)
        gate_up_ms = [gate_up_avg] * (args.steps * LAYERS)
        gate_up_bytes = 2 * gemv_bytes(HIDDEN, DIM)

        ms = min(ms_step, ms_step_clean)
        gbs = total_bytes / (ms * 1e-3) / 1e9
        achieved = gate_up_bytes / (gate_up_avg * 1e-3) / 1e9
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
                       "bytes_per_step": total_bytes, "device": name, "compute_units": cu},
            "frac_hbm_peak": round(gbs / HBM_PEAK_GBS, 4),
            "tok_s": round(1e3 / ms, 1),
            "ms_per_step_graph": round(ms_step_clean, 4),
            "ms_per_step_python_launches": round(ms_step, 4),
            "host_wall_ms_per_step": round(wall * 1e3 / args.steps, 4),
            "roofline": {"bound": "hbm", "kernel": "jl_gemv_tiles<Q8_0, gate/up> 2 x [8192 x 2048]",
                         "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                         "frac": round(achieved / HBM_PEAK_GBS, 4), "traffic": GATE_UP_HBM_TRAFFIC_BYTES,
                         "bytes_per_launch": gate_up_bytes,
                         "avg_launch_us": round(gate_up_avg * 1e3, 3),
                         "launches_timed": len(gate_up_ms)},
        }
        legs = set() if args.no_extra else set(args.extra.split(","))
        if "fused_rms" in legs:
            out["decode_fused_rms"] = bench_fused_rms(ctx, hip, proj, layers, wcls, acts, args.steps,
                                                      args.warmup)
        if "prefill" in legs:
            # (the matrix pipe's clock takes tens of milliseconds of load to settle: 100 untimed
            # replays of the layer before the timed ones)
            out["prefill"] = [bench_gemm(ctx, hip, t, T, args.steps, 100) for T in (512, 2048)]
        if "other_types" in legs:
            out["decode_other_types"] = [
                bench_decode_layers(ctx, hip, "Q4_0", 4096, 1024, 14336, 4, args.steps, args.warmup),
                bench_decode_layers(ctx, hip, "Q4_K", 4096, 1024, 12288, 4, args.steps, args.warmup)]
        if "batched" in legs:
            out["batched_q4k"] = [bench_batched_q4k(ctx, hip, B, max(5, args.steps // 5), 3)
                                  for B in (8, 32, 64)]
        if not args.no_cpu:
            out["cpu_baseline"] = cpu_baseline(host, shapes, t)
        else:
            out["cpu_baseline"] = None
    print(json.dumps(out))


if __name__ == "__main__":
    main()
