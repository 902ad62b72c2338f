"""GPU parity of the batched prefill over fp16 activations (jl_gemm_xf16): the operand types the
reference's prefill GEMMs take (fp16 in, fp32 out; the feed-forward hidden vector fp16 out).  Pinned
three ways: to the fp32 entry point bit for bit on inputs fp16 holds exactly, to the oracle on the
widened inputs, and -- the fp16 output -- to the fp32 output rounded once."""
import ctypes as C

import numpy as np
import pytest

from gpu_util import magnitude, rel_err, say
from oracle import pyoracle as O

pytestmark = pytest.mark.gpu

F16_BOUND = 2e-3                  # fp16-MFMA path: max |d| / sum |w x|
UNTOUCHED = np.float32(-12345.5)


@pytest.fixture(scope="module")
def ctx():
    from jitllm_amd.runtime import Context
    c = Context(0)
    yield c
    c.close()


def half_activations(shape, seed):
    from jitllm_amd import synthetic
    return synthetic.activations(shape, seed=seed).astype(np.float16)


# (type, weight rows, row length, batch, active rows, residual): whole-tile batches read in place by
# the decode-once path (one with K cut in two), ragged ones copied into the workspace, small ones
# on the decode-in-the-loop kernel, and a type that always decodes once
CASES = [
    (O.Q8_0, 3072, 2048, 512, 512, False),
    (O.Q8_0, 2048, 2048, 2048, 2048, True),
    (O.Q4_K, 4100, 1024, 600, 600, False),
    (O.Q4_K, 4100, 1024, 768, 600, True),
    (O.Q4_0, 1000, 512, 130, 130, True),
    (O.Q8_0, 300, 256, 9, 9, False),
    (O.Q8_0, 300, 256, 64, 40, True),
    (O.Q8_0, 300, 256, 96, 70, True),
    (O.Q6_K, 640, 512, 96, 90, False),
    (O.Q4_K, 4100, 4096, 32, 32, True),      # up to 64 rows: the weight-streaming kernel, rows cut across workgroups
    (O.Q4_0, 1000, 2048, 64, 50, False),
    (O.IQ4_XS, 520, 1024, 16, 16, True),
]


@pytest.mark.parametrize("t,d,n,batch,rows,residual", CASES)
def test_fp16_activations_give_the_fp32_entry_points_bits(ctx, t, d, n, batch, rows, residual):
    from jitllm_amd import synthetic
    from jitllm_amd.projections import QuantizedBatchProjections
    say("xf16 projection", t, d, n, batch, rows, residual)
    raw = synthetic.weight(t, d, n, seed=1700 + d % 97)
    w = ctx.load_weight(t, raw, d, n)
    X16 = half_activations((batch, n), 1701)
    X32 = X16.astype(np.float32)
    start = synthetic.activations((batch, d), seed=1702) if residual else np.full((batch, d), UNTOUCHED, np.float32)
    p = QuantizedBatchProjections(ctx, batch, n, d)
    a, b = ctx.from_numpy(start), ctx.from_numpy(start)
    p.projection(ctx.from_numpy(X32), a, w, n, d, residual, activeRows=rows)
    p.projection(ctx.half_from_numpy(X16), b, w, n, d, residual, activeRows=rows)
    ctx.sync()
    got32, got16 = a.get().reshape(batch, d), b.get().reshape(batch, d)
    assert np.array_equal(got16.view(np.uint32), got32.view(np.uint32))
    assert np.array_equal(got16[rows:], start[rows:])
    ref = O.matmul_batch(t, raw, X32[:rows], d, n).astype(np.float64) + (start[:rows] if residual else 0.0)
    mag = magnitude(t, raw, X32[:rows], d, n) + (np.abs(start[:rows]) * 1e-6 if residual else 0.0)
    assert rel_err(got16[:rows], ref, mag) < F16_BOUND


# (the last two: 3072 and 6144 columns on 128 x 192 and 256 x 192 tiles, whose column tiles straddle
# the three weights' boundaries; ragged rows in the second)
@pytest.mark.parametrize("t,dq,dkv,n,T,resident", [(O.Q8_0, 2048, 512, 2048, 512, True), (O.Q4_K, 256, 128, 1024, 70, False),
                                                   (O.Q8_0, 2048, 512, 256, 2048, True), (O.Q4_0, 4096, 1024, 256, 2000, False)])
def test_fp16_activations_fused_qkv(ctx, t, dq, dkv, n, T, resident):
    from jitllm_amd import synthetic
    from jitllm_amd.projections import QuantizedBatchProjections
    say("xf16 qkv", t, T)
    raws = [synthetic.weight(t, r, n, seed=1710 + i) for i, r in enumerate((dq, dkv, dkv))]
    ws = [ctx.load_weight(t, raw, r, n) for raw, r in zip(raws, (dq, dkv, dkv))]
    X16 = half_activations((T, n), 1713)
    width = dq + 2 * dkv
    p = QuantizedBatchProjections(ctx, T, n, width, resident=resident)
    a, b = ctx.float_array(T * width, fill=UNTOUCHED), ctx.float_array(T * width, fill=UNTOUCHED)
    for _ in range(2):                                   # the second call reuses the resident copy
        p.fusedQKV(ctx.from_numpy(X16.astype(np.float32)), a, *ws)
        p.fusedQKV(ctx.half_from_numpy(X16), b, *ws)
        ctx.sync()
        got = b.get().reshape(T, width)
        assert np.array_equal(got.view(np.uint32), a.get().reshape(T, width).view(np.uint32))
    col = 0
    for raw, r in zip(raws, (dq, dkv, dkv)):
        ref = O.matmul_batch(t, raw, X16.astype(np.float32), r, n)
        assert rel_err(got[:, col:col + r], ref, magnitude(t, raw, X16.astype(np.float32), r, n)) < F16_BOUND
        col += r


@pytest.mark.parametrize("t,ffn,n,batch,rows", [(O.Q8_0, 8192, 2048, 512, 512), (O.Q4_K, 1002, 512, 768, 700),
                                                (O.Q4_0, 1002, 1024, 96, 96), (O.Q5_K, 520, 256, 96, 70),
                                                (O.Q4_K, 1002, 4096, 40, 33), (O.Q8_0, 520, 2048, 64, 64),
                                                (O.Q6_K, 300, 2048, 8, 5)])
def test_fp16_hidden_vector_is_the_fp32_one_rounded_once(ctx, t, ffn, n, batch, rows):
    """gate/up + SwiGLU with the result stored as fp16 (batchedFFNSwiGLUFP16Packed): every value is
    the fp32 result of the same call rounded to nearest even, rows past the active ones untouched;
    the fp32 result itself equals the fp32 entry point's and meets the oracle.  (The last three:
    at most 64 rows, where both kinds of activations take the weight-streaming kernel -- a short
    prompt's prefill.)"""
    from jitllm_amd import synthetic
    from jitllm_amd.projections import QuantizedBatchProjections
    say("xf16 gate/up", t, ffn, n, batch, rows)
    r1, r3 = synthetic.weight(t, ffn, n, seed=1720), synthetic.weight(t, ffn, n, seed=1721)
    w1, w3 = ctx.load_weight(t, r1, ffn, n), ctx.load_weight(t, r3, ffn, n)
    X16 = half_activations((batch, n), 1722)
    X32 = X16.astype(np.float32)
    p = QuantizedBatchProjections(ctx, batch, n, 2 * ffn)
    h32, h32x = ctx.float_array(batch * ffn, fill=UNTOUCHED), ctx.float_array(batch * ffn, fill=UNTOUCHED)
    h16 = ctx.half_from_numpy(np.full(batch * ffn, 7.5, dtype=np.float16))
    dx = ctx.half_from_numpy(X16)
    # (called below the mirror's gateUp, which keeps the reference's rule that only Q8_0 / Q4_0 /
    # Q4_K pairs are fused; the library takes the Q5_K pair)
    from jitllm_amd import _lib as L
    p._gemm([w1, w3], ctx.from_numpy(X32), h32, rows, ffn, 0, L.JL_SWIGLU)
    p._gemm([w1, w3], dx, h32x, rows, ffn, 0, L.JL_SWIGLU)
    p._gemm([w1, w3], dx, h16, rows, ffn, 0, L.JL_SWIGLU)
    ctx.sync()
    a, b, c = h32.get().reshape(batch, ffn), h32x.get().reshape(batch, ffn), h16.get().reshape(batch, ffn)
    assert np.array_equal(a.view(np.uint32), b.view(np.uint32))
    assert np.array_equal(c[:rows].view(np.uint16), b[:rows].astype(np.float16).view(np.uint16))
    assert np.all(c[rows:] == np.float16(7.5))
    g = O.matmul_batch(t, r1, X32[:rows], ffn, n)
    u = O.matmul_batch(t, r3, X32[:rows], ffn, n)
    want = O.swiglu(g.reshape(-1), u.reshape(-1)).reshape(rows, ffn)
    mg, mu = magnitude(t, r1, X32[:rows], ffn, n), magnitude(t, r3, X32[:rows], ffn, n)
    bound = F16_BOUND * (mg * np.abs(u) + 1.2 * mu * np.abs(g)) + 1e-6
    assert np.all(np.abs(b[:rows].astype(np.float64) - want) <= bound)


def test_fp16_hidden_vector_at_an_odd_offset(ctx):
    """ldo and col_offset count fp16 values; an output row that starts on an odd element takes the
    element-wise stores and leaves its neighbours alone."""
    from jitllm_amd import _lib as L, synthetic
    from jitllm_amd.projections import QuantizedBatchProjections
    say("xf16 gate/up offset")
    t, ffn, n, T, ldo, off = O.Q8_0, 130, 256, 40, 141, 3
    r1, r3 = synthetic.weight(t, ffn, n, seed=1730), synthetic.weight(t, ffn, n, seed=1731)
    w1, w3 = ctx.load_weight(t, r1, ffn, n), ctx.load_weight(t, r3, ffn, n)
    dx = ctx.half_from_numpy(half_activations((T, n), 1732))
    p = QuantizedBatchProjections(ctx, T, n, 2 * ffn)
    h32 = ctx.float_array(T * ffn)
    h16 = ctx.half_from_numpy(np.full(T * ldo, 7.5, dtype=np.float16))
    p.gateUp(dx, h32, w1, w3, n, ffn)
    arr = (C.c_void_p * 2)(w1.handle, w3.handle)
    L.check(ctx._lib.jl_gemm_xf16(ctx.handle, arr, 2, dx.ptr, h16.ptr, 1, T, T, ldo, off, L.JL_SWIGLU,
                                  p.workspace.ptr, p.workspace.nbytes, None, 0, None))
    ctx.sync()
    got = h16.get().reshape(T, ldo)
    assert np.array_equal(got[:, off:off + ffn].view(np.uint16),
                          h32.get().reshape(T, ffn).astype(np.float16).view(np.uint16))
    assert np.all(got[:, :off] == np.float16(7.5)) and np.all(got[:, off + ffn:] == np.float16(7.5))


def test_plugin_instance_takes_the_references_operand_types(ctx):
    """A layer's steps through the plugin mirror with fp16 activations in, fp32 out and an fp16
    hidden vector feeding the down projection, against the oracle on the same fp16 values."""
    from jitllm_amd import ops, synthetic
    from jitllm_amd.ggml import GGMLType
    from jitllm_amd.ops import HipImplementation, MatMul, ResidualAdd, SwiGLU, Target, TensorRole as R
    say("xf16 plugin layer")
    t, T, dim, kv, ffn = O.Q8_0, 512, 512, 256, 4352
    g = GGMLType(t)
    shapes = {R.ATTENTION_QUERY: (dim, dim), R.ATTENTION_KEY: (kv, dim), R.ATTENTION_VALUE: (kv, dim),
              R.FFN_GATE: (ffn, dim), R.FFN_UP: (ffn, dim), R.FFN_DOWN: (dim, ffn)}
    raws = {r: synthetic.weight(g, d, n, seed=1740 + i) for i, (r, (d, n)) in enumerate(shapes.items())}
    tensors = {r: ctx.load_weight(g, raws[r], *shapes[r]) for r in shapes}
    program = [
        MatMul(R.ATTENTION_QUERY, "xb", "qkv", dim, dim, T, g), MatMul(R.ATTENTION_KEY, "xb", "k", kv, dim, T, g),
        MatMul(R.ATTENTION_VALUE, "xb", "v", kv, dim, T, g),
        MatMul(R.FFN_GATE, "xb", "hb", ffn, dim, T, g), MatMul(R.FFN_UP, "xb", "hb2", ffn, dim, T, g),
        SwiGLU("hb", "hb2", "hb"),
        MatMul(R.FFN_DOWN, "hb", "xb2", dim, ffn, T, g), ResidualAdd("x", "xb2"),
    ]
    impl = HipImplementation(residency=True)
    steps = [c.step for c in ops.split(program, 0, T, [impl], Target())]
    xb = half_activations((T, dim), 1750)
    x = synthetic.activations((T, dim), 1751)
    acts = {"xb": ctx.half_from_numpy(xb), "x": ctx.from_numpy(x), "qkv": ctx.float_array(T * (dim + 2 * kv)),
            "hb": ctx.half_array(T * ffn)}
    inst = impl.create(steps, Target(), ctx)
    operands = ops.Operands(acts, lambda role, layer: tensors[role])
    for step in steps:
        inst.emit(step, operands)
    ctx.sync()
    xb32 = xb.astype(np.float32)
    got = acts["qkv"].get().reshape(T, dim + 2 * kv)
    col = 0
    for r in (R.ATTENTION_QUERY, R.ATTENTION_KEY, R.ATTENTION_VALUE):
        d, n = shapes[r]
        assert rel_err(got[:, col:col + d], O.matmul_batch(t, raws[r], xb32, d, n), magnitude(t, raws[r], xb32, d, n)) < F16_BOUND
        col += d
    hb = acts["hb"].get().reshape(T, ffn)
    gt, up = O.matmul_batch(t, raws[R.FFN_GATE], xb32, ffn, dim), O.matmul_batch(t, raws[R.FFN_UP], xb32, ffn, dim)
    want = O.swiglu(gt.reshape(-1), up.reshape(-1)).reshape(T, ffn)
    mg, mu = magnitude(t, raws[R.FFN_GATE], xb32, ffn, dim), magnitude(t, raws[R.FFN_UP], xb32, ffn, dim)
    bound = F16_BOUND * (mg * np.abs(up) + 1.2 * mu * np.abs(gt)) + np.abs(want) * 2.0 ** -11 + 1e-6
    assert np.all(np.abs(hb.astype(np.float64) - want) <= bound)
    # the down projection read exactly the fp16 hidden vector the device holds
    hb32 = hb.astype(np.float32)
    ref = O.matmul_batch(t, raws[R.FFN_DOWN], hb32, dim, ffn).astype(np.float64) + x
    mag = magnitude(t, raws[R.FFN_DOWN], hb32, dim, ffn) + np.abs(x) * 1e-6
    assert rel_err(acts["x"].get().reshape(T, dim), ref, mag) < F16_BOUND


def test_plugin_instance_runs_the_whole_layer_plan(ctx):
    """Every step of the reference's tensor-core table through the plugin mirror, in a Llama layer's
    order: RMS norm -> q|k|v, o projection, residual add + RMS norm -> gate|up + SwiGLU, down +
    residual add (TensorCoreSteps.java:44-78, 133-169), and the bare residual add behind a down
    projection.  The norms are held to the oracle bit for bit (fp16 rows and row scales), the
    projections to the oracle on exactly the fp16 rows the device holds."""
    from jitllm_amd import ops, synthetic
    from jitllm_amd.ggml import GGMLType
    from jitllm_amd.ops import (ADD_NORM, DOWN_ADD, GATE_UP_SWIGLU, NORM, PROJECTION, QKV, RESIDUAL, HipImplementation,
                                MatMul, ResidualAdd, RmsNorm, Step, SwiGLU, Target, TensorRole as R)
    say("whole layer plan")
    t, T, dim, kv, ffn, eps = O.Q4_K, 200, 512, 256, 1536, 1e-5
    g = GGMLType(t)
    shapes = {R.ATTENTION_QUERY: (dim, dim), R.ATTENTION_KEY: (kv, dim), R.ATTENTION_VALUE: (kv, dim),
              R.ATTENTION_OUTPUT: (dim, dim), R.FFN_GATE: (ffn, dim), R.FFN_UP: (ffn, dim), R.FFN_DOWN: (dim, ffn)}
    raws = {r: synthetic.weight(g, d, n, seed=1770 + i) for i, (r, (d, n)) in enumerate(shapes.items())}
    tensors = {r: ctx.load_weight(g, raws[r], *shapes[r]) for r in shapes}
    norm_w = {R.ATTENTION_NORM: np.random.default_rng(1780).uniform(0.5, 1.5, dim).astype(np.float32),
              R.FFN_NORM: np.random.default_rng(1781).uniform(0.5, 1.5, dim).astype(np.float32)}
    tensors.update({r: ctx.from_numpy(w) for r, w in norm_w.items()})
    down = MatMul(R.FFN_DOWN, "hb", "xb2", dim, ffn, T, g)
    program = [
        RmsNorm("x", "xb", R.ATTENTION_NORM, eps, dim),
        MatMul(R.ATTENTION_QUERY, "xb", "qkv", dim, dim, T, g), MatMul(R.ATTENTION_KEY, "xb", "k", kv, dim, T, g),
        MatMul(R.ATTENTION_VALUE, "xb", "v", kv, dim, T, g),
        MatMul(R.ATTENTION_OUTPUT, "att", "xb2", dim, dim, T, g),
        ResidualAdd("x", "xb2"), RmsNorm("x", "xb", R.FFN_NORM, eps, dim),
        MatMul(R.FFN_GATE, "xb", "hb", ffn, dim, T, g), MatMul(R.FFN_UP, "xb", "hb2", ffn, dim, T, g),
        SwiGLU("hb", "hb2", "hb"),
        down, ResidualAdd("x", "xb2"),
    ]
    impl = HipImplementation()
    chosen = ops.split(program, 0, T, [impl], Target())
    assert [c.step.fusion.name for c in chosen] == [NORM.name, QKV.name, PROJECTION.name, ADD_NORM.name,
                                                    GATE_UP_SWIGLU.name, DOWN_ADD.name]
    steps = [c.step for c in chosen]
    x0 = synthetic.activations((T, dim), 1790) * np.float32(1.7)
    att = half_activations((T, dim), 1791)
    acts = {"x": ctx.from_numpy(x0), "xb": ctx.half_array(T * dim), "xb.scale": ctx.float_array(T, fill=UNTOUCHED),
            "att": ctx.half_from_numpy(att), "xb2": ctx.float_array(T * dim), "qkv": ctx.float_array(T * (dim + 2 * kv)),
            "hb": ctx.half_array(T * ffn)}
    operands = ops.Operands(acts, lambda role, layer: tensors[role])
    inst = impl.create(steps, Target(), ctx)

    def held_to(name, got, raw_role, X32):
        d, n = shapes[raw_role]
        assert rel_err(got, O.matmul_batch(t, raws[raw_role], X32, d, n), magnitude(t, raws[raw_role], X32, d, n)) < F16_BOUND, name

    # RMS norm -> q|k|v
    inst.emit(steps[0], operands)
    inst.emit(steps[1], operands)
    ctx.sync()
    want_scale, want_xb = O.batched_rms_apply_f16(x0, norm_w[R.ATTENTION_NORM], eps)
    xb = acts["xb"].get().reshape(T, dim)
    assert np.array_equal(xb.view(np.uint16), want_xb.view(np.uint16))
    assert np.array_equal(acts["xb.scale"].get().view(np.uint32), want_scale.view(np.uint32))
    assert np.array_equal(acts["x"].get().reshape(T, dim), x0)          # a norm on its own only reads x
    qkv = acts["qkv"].get().reshape(T, dim + 2 * kv)
    col = 0
    for r in (R.ATTENTION_QUERY, R.ATTENTION_KEY, R.ATTENTION_VALUE):
        held_to(r, qkv[:, col:col + shapes[r][0]], r, xb.astype(np.float32))
        col += shapes[r][0]
    # o projection, then the residual add inside the next norm
    inst.emit(steps[2], operands)
    ctx.sync()
    xb2 = acts["xb2"].get().reshape(T, dim)
    held_to("o", xb2, R.ATTENTION_OUTPUT, att.astype(np.float32))
    inst.emit(steps[3], operands)
    ctx.sync()
    x1 = x0 + xb2
    assert np.array_equal(acts["x"].get().reshape(T, dim).view(np.uint32), x1.view(np.uint32))
    want_scale, want_xb = O.batched_rms_apply_f16(x1, norm_w[R.FFN_NORM], eps)
    xb = acts["xb"].get().reshape(T, dim)
    assert np.array_equal(xb.view(np.uint16), want_xb.view(np.uint16))
    assert np.array_equal(acts["xb.scale"].get().view(np.uint32), want_scale.view(np.uint32))
    # gate|up + SwiGLU into the fp16 hidden rows, down + residual add
    inst.emit(steps[4], operands)
    inst.emit(steps[5], operands)
    ctx.sync()
    xb32 = xb.astype(np.float32)
    hb = acts["hb"].get().reshape(T, ffn)
    gt, up = O.matmul_batch(t, raws[R.FFN_GATE], xb32, ffn, dim), O.matmul_batch(t, raws[R.FFN_UP], xb32, ffn, dim)
    want = O.swiglu(gt.reshape(-1), up.reshape(-1)).reshape(T, ffn)
    mg, mu = magnitude(t, raws[R.FFN_GATE], xb32, ffn, dim), magnitude(t, raws[R.FFN_UP], xb32, ffn, dim)
    assert np.all(np.abs(hb.astype(np.float64) - want) <= F16_BOUND * (mg * np.abs(up) + 1.2 * mu * np.abs(gt))
                  + np.abs(want) * 2.0 ** -11 + 1e-6)
    hb32 = hb.astype(np.float32)
    ref = O.matmul_batch(t, raws[R.FFN_DOWN], hb32, dim, ffn).astype(np.float64) + x1
    mag = magnitude(t, raws[R.FFN_DOWN], hb32, dim, ffn) + np.abs(x1) * 1e-6
    x2 = acts["x"].get().reshape(T, dim)
    assert rel_err(x2, ref, mag) < F16_BOUND
    # the down projection and its residual add as two steps (a family with a task of its own between them)
    inst.emit(Step(0, T, PROJECTION, (down,)), operands)
    inst.emit(Step(0, T, RESIDUAL, (ResidualAdd("x", "xb2"),)), operands)
    ctx.sync()
    assert np.array_equal(acts["x"].get().reshape(T, dim).view(np.uint32),
                          (x2 + acts["xb2"].get().reshape(T, dim)).view(np.uint32))
    # ... and a bare add that follows anything else is refused by name
    inst.emit(Step(0, T, PROJECTION, (MatMul(R.ATTENTION_OUTPUT, "att", "xb2", dim, dim, T, g),)), operands)
    with pytest.raises(ValueError, match="follows the down projection, not xb2"):
        inst.emit(Step(0, T, RESIDUAL, (ResidualAdd("x", "xb2"),)), operands)
    ctx.sync()


def test_xf16_refusals(ctx):
    from jitllm_amd import _lib as L, synthetic
    from jitllm_amd.projections import QuantizedBatchProjections
    say("xf16 refusals")
    t, d, n, T = O.Q8_0, 64, 256, 8
    w = ctx.load_weight(t, synthetic.weight(t, d, n, seed=1760), d, n)
    p = QuantizedBatchProjections(ctx, T, n, d)
    dx = ctx.half_from_numpy(half_activations((T, n), 1761))
    with pytest.raises(L.JitllmHipError, match="only the JL_SWIGLU result"):
        p.projection(dx, ctx.half_array(T * d), w, n, d, False)
    with pytest.raises(ValueError, match="fp16 output needs fp16 activations"):
        p.projection(ctx.float_array(T * n), ctx.half_array(T * d), w, n, d, False)
    arr = (C.c_void_p * 1)(w.handle)
    out = ctx.float_array(T * d)
    copy = ctx.raw_buffer(1 << 20)
    with pytest.raises(L.JitllmHipError, match="go together"):
        L.check(ctx._lib.jl_gemm_xf16(ctx.handle, arr, 1, dx.ptr, out.ptr, 0, T, T, d, 0, L.JL_STORE,
                                      p.workspace.ptr, p.workspace.nbytes, copy.ptr, copy.nbytes, None))
    with pytest.raises(L.JitllmHipError, match="null argument"):
        L.check(ctx._lib.jl_gemm_xf16(ctx.handle, arr, 1, None, out.ptr, 0, T, T, d, 0, L.JL_STORE,
                                      p.workspace.ptr, p.workspace.nbytes, None, 0, None))


@pytest.mark.parametrize("rows,n", [(1, 2048), (70, 2048), (600, 1000), (33, 8192), (5, 8448), (3, 16384)])
def test_rms_apply_to_fp16_has_the_oracles_bits(ctx, rows, n):
    """batchedRmsReduceParallel + batchedRmsApplyFP16 in one launch: the kernel sums in the
    reference kernel's own order, so scales and fp16 outputs equal the oracle's bit for bit (rows
    held in registers up to 8192 columns, re-read beyond; a row length that is no multiple of 256)."""
    from jitllm_amd import synthetic
    from jitllm_amd.projections import QuantizedBatchProjections
    say("rms apply fp16", rows, n)
    x = synthetic.activations((rows, n), seed=1800 + n) * np.float32(2.5)
    x[0, :7] = [0.0, -0.0, 1e-30, 3e4, -3e4, 65504.0, 1e-8]
    w = np.random.default_rng(1801).uniform(0.5, 1.5, n).astype(np.float32)
    p = QuantizedBatchProjections(ctx, rows + 2, 256, 256)
    out = ctx.half_from_numpy(np.full((rows + 2) * n, 7.5, dtype=np.float16))
    scales = ctx.float_array(rows + 2, fill=UNTOUCHED)
    p.rmsApplyFP16(ctx.from_numpy(np.concatenate([x, np.zeros((2, n), np.float32)])), ctx.from_numpy(w), 1e-5, out, n,
                   scales=scales, activeRows=rows)
    ctx.sync()
    want_scales, want = O.batched_rms_apply_f16(x, w, 1e-5)
    got_scales, got = scales.get(), out.get().reshape(rows + 2, n)
    assert np.array_equal(got_scales[:rows].view(np.uint32), want_scales.view(np.uint32))
    assert np.all(got_scales[rows:] == UNTOUCHED)
    assert np.array_equal(got[:rows].view(np.uint16), want.view(np.uint16))
    assert np.all(got[rows:] == np.float16(7.5))


def test_normalise_then_project_in_fp16(ctx):
    """The prefill plan's first two steps chained on the device -- RMS apply to fp16, then q|k|v over
    the fp16 rows -- against the oracle's projection of the oracle's fp16 activations."""
    from jitllm_amd import synthetic
    from jitllm_amd.projections import QuantizedBatchProjections
    say("rms apply fp16 -> qkv")
    t, T, n, dq, dkv = O.Q8_0, 512, 2048, 2048, 512
    raws = [synthetic.weight(t, r, n, seed=1810 + i) for i, r in enumerate((dq, dkv, dkv))]
    ws = [ctx.load_weight(t, raw, r, n) for raw, r in zip(raws, (dq, dkv, dkv))]
    x = synthetic.activations((T, n), seed=1813) * np.float32(4.0)
    w = np.random.default_rng(1814).uniform(0.5, 1.5, n).astype(np.float32)
    p = QuantizedBatchProjections(ctx, T, n, dq + 2 * dkv)
    xb16 = ctx.half_array(T * n)
    qkv = ctx.float_array(T * (dq + 2 * dkv), fill=UNTOUCHED)
    p.rmsApplyFP16(ctx.from_numpy(x), ctx.from_numpy(w), 1e-5, xb16, n)
    p.fusedQKV(xb16, qkv, *ws)
    ctx.sync()
    _, xb = O.batched_rms_apply_f16(x, w, 1e-5)
    xb32 = xb.astype(np.float32)
    got = qkv.get().reshape(T, dq + 2 * dkv)
    col = 0
    for raw, r in zip(raws, (dq, dkv, dkv)):
        assert rel_err(got[:, col:col + r], O.matmul_batch(t, raw, xb32, r, n), magnitude(t, raw, xb32, r, n)) < F16_BOUND
        col += r


@pytest.mark.parametrize("rows,n", [(40, 2048), (7, 3000), (3, 8448)])
def test_rms_apply_with_the_pending_residual(ctx, rows, n):
    """batchedRmsReduceFusedResidual folded in: x += delta is written back (active rows only) and
    scales and fp16 outputs are the oracle's for the updated rows, bit for bit."""
    from jitllm_amd import synthetic
    from jitllm_amd.projections import QuantizedBatchProjections
    say("rms apply fp16 + residual", rows, n)
    x = synthetic.activations((rows + 1, n), seed=1900 + n)
    delta = synthetic.activations((rows + 1, n), seed=1901 + n) * np.float32(0.25)
    w = np.random.default_rng(1902).uniform(0.5, 1.5, n).astype(np.float32)
    p = QuantizedBatchProjections(ctx, rows + 1, 256, 256)
    dx, out, scales = ctx.from_numpy(x), ctx.half_array((rows + 1) * n), ctx.float_array(rows + 1)
    p.rmsApplyFP16(dx, ctx.from_numpy(w), 1e-5, out, n, scales=scales, activeRows=rows, delta=ctx.from_numpy(delta))
    ctx.sync()
    updated = []
    want_scales, want = O.batched_rms_apply_f16(x[:rows], w, 1e-5, delta=delta[:rows], updated=updated)
    got_x = dx.get().reshape(rows + 1, n)
    assert np.array_equal(got_x[:rows].view(np.uint32), updated[0].view(np.uint32))
    assert np.array_equal(got_x[rows], x[rows])
    assert np.array_equal(scales.get()[:rows].view(np.uint32), want_scales.view(np.uint32))
    assert np.array_equal(out.get().reshape(rows + 1, n)[:rows].view(np.uint16), want.view(np.uint16))
