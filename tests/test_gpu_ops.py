"""GPU: the plugin instance runs a layer's projection steps like the host's matmul sequence."""
import numpy as np
import pytest

from gpu_util import magnitude, rel_err, say
from oracle import pyoracle as O

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ctx():
    from jitllm_amd.runtime import Context
    c = Context(0)
    yield c
    c.close()


# "Q4_K_M": a layer as such a file holds it -- Q4_K except the value and down projections in Q6_K, so
# that q|k|v is one step over two types; "odd pair": a gate and an up weight of different types
@pytest.mark.parametrize("t,T,residency", [(O.Q8_0, 40, False), (O.Q4_K, 600, False), (O.Q4_K, 600, True),
                                           (O.Q6_K, 40, True), ("Q4_K_M", 40, False), ("Q4_K_M", 600, True),
                                           ("odd pair", 130, False)])
def test_instance_emits_a_layer(ctx, t, T, residency):
    from jitllm_amd import ops, synthetic
    from jitllm_amd.ggml import GGMLType
    from jitllm_amd.ops import HipImplementation, MatMul, ResidualAdd, SwiGLU, Target, TensorRole as R
    say("ops layer", t, T, residency)
    dim, kv, ffn = 512, 256, 4352
    mixed = {"Q4_K_M": {R.ATTENTION_VALUE: O.Q6_K, R.FFN_DOWN: O.Q6_K}, "odd pair": {R.FFN_UP: O.Q5_0}}.get(t, {})
    base = O.Q4_K if isinstance(t, str) else t
    shapes = {R.ATTENTION_QUERY: (dim, dim), R.ATTENTION_KEY: (kv, dim), R.ATTENTION_VALUE: (kv, dim),
              R.ATTENTION_OUTPUT: (dim, dim), R.FFN_GATE: (ffn, dim), R.FFN_UP: (ffn, dim), R.FFN_DOWN: (dim, ffn)}
    tt = {r: mixed.get(r, base) for r in shapes}          # the type of each role's weight
    g = {r: GGMLType(tt[r]) for r in shapes}
    raws = {r: synthetic.weight(g[r], d, n, seed=1000 + i) for i, (r, (d, n)) in enumerate(shapes.items())}
    tensors = {r: ctx.load_weight(g[r], raws[r], *shapes[r]) for r in shapes}
    program = [
        MatMul(R.ATTENTION_QUERY, "xb", "qkv", dim, dim, T, g[R.ATTENTION_QUERY]),
        MatMul(R.ATTENTION_KEY, "xb", "k", kv, dim, T, g[R.ATTENTION_KEY]),
        MatMul(R.ATTENTION_VALUE, "xb", "v", kv, dim, T, g[R.ATTENTION_VALUE]),
        MatMul(R.ATTENTION_OUTPUT, "att", "xb2", dim, dim, T, g[R.ATTENTION_OUTPUT]),
        MatMul(R.FFN_GATE, "xb", "hb", ffn, dim, T, g[R.FFN_GATE]), MatMul(R.FFN_UP, "xb", "hb2", ffn, dim, T, g[R.FFN_UP]),
        SwiGLU("hb", "hb2", "hb"),
        MatMul(R.FFN_DOWN, "hb_in", "xb2", dim, ffn, T, g[R.FFN_DOWN]), ResidualAdd("x", "xb2"),
    ]
    impl = HipImplementation(residency=residency)
    chosen = ops.split(program, 0, T, [impl], Target())
    if t == O.Q6_K or isinstance(t, str):
        # no fused gate|up + SwiGLU restriction applies to jl_gemm, and the weights of a step may
        # differ in type: the steps are claimed whole
        assert [c.step.fusion.name for c in chosen] == ["q|k|v", "projection", "gate|up + SwiGLU", "down + residual add"]
    steps = [c.step for c in chosen]
    host = {"xb": synthetic.activations((T, dim), 1101), "att": synthetic.activations((T, dim), 1102),
            "hb_in": synthetic.activations((T, ffn), 1103) * np.float32(0.1),
            "x": synthetic.activations((T, dim), 1104)}
    acts = {k: ctx.from_numpy(v) for k, v in host.items()}
    acts.update({"qkv": ctx.float_array(T * (dim + 2 * kv)), "xb2": ctx.float_array(T * dim),
                 "hb": ctx.float_array(T * ffn)})
    operands = ops.Operands(acts, lambda role, layer: tensors[role])
    need = impl.needs(steps, Target())
    inst = impl.create(steps, Target(), ctx)
    assert inst.buffers()[0].nbytes == max(need.bytes, 256)
    narrow = impl.narrowed(inst, steps, Target(), ctx)
    for round_ in range(2):                     # the second pass reuses resident copies
        acts["x"].set(host["x"].reshape(-1))
        for step in steps:
            (narrow if round_ else inst).emit(step, operands)
        ctx.sync()
        tol = 5e-4
        got = acts["qkv"].get().reshape(T, dim + 2 * kv)
        col = 0
        for r in (R.ATTENTION_QUERY, R.ATTENTION_KEY, R.ATTENTION_VALUE):
            d, n = shapes[r]
            ref = O.matmul_batch(tt[r], raws[r], host["xb"], d, n)
            assert rel_err(got[:, col:col + d], ref, magnitude(tt[r], raws[r], host["xb"], d, n)) < tol
            col += d
        ref = O.matmul_batch(tt[R.ATTENTION_OUTPUT], raws[R.ATTENTION_OUTPUT], host["att"], dim, dim)
        assert rel_err(acts["xb2"].get().reshape(T, dim), ref,
                       magnitude(tt[R.ATTENTION_OUTPUT], raws[R.ATTENTION_OUTPUT], host["att"], dim, dim)) < tol
        gt = O.matmul_batch(tt[R.FFN_GATE], raws[R.FFN_GATE], host["xb"], ffn, dim)
        up = O.matmul_batch(tt[R.FFN_UP], raws[R.FFN_UP], host["xb"], ffn, dim)
        want = O.swiglu(gt.reshape(-1), up.reshape(-1)).reshape(T, ffn)
        mg = magnitude(tt[R.FFN_GATE], raws[R.FFN_GATE], host["xb"], ffn, dim)
        mu = magnitude(tt[R.FFN_UP], raws[R.FFN_UP], host["xb"], ffn, dim)
        bound = tol * (mg * np.abs(up) + 1.2 * mu * np.abs(gt)) + 1e-6
        assert np.all(np.abs(acts["hb"].get().reshape(T, ffn).astype(np.float64) - want) <= bound)
        ref = O.matmul_batch(tt[R.FFN_DOWN], raws[R.FFN_DOWN], host["hb_in"], dim, ffn).astype(np.float64) + host["x"]
        mag = magnitude(tt[R.FFN_DOWN], raws[R.FFN_DOWN], host["hb_in"], dim, ffn) + np.abs(host["x"]) * 1e-6
        assert rel_err(acts["x"].get().reshape(T, dim), ref, mag) < tol
    if residency:
        assert len(inst.copies) == len(steps) and narrow.copies is inst.copies
