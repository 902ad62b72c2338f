"""Committed vectors (tests/golden/).  projection_golden.npz is a freeze of the oracle -- inputs from
the reference's test recipes, outputs written by oracle/ itself (make_golden.py) -- not a vector
the reference holds: the oracle must keep reproducing it bit for bit on the CPU, and the HIP library
must match it on the GPU without the oracle recomputing anything.  reference_known_answers.json is
the one file of answers the reference itself states (Q4_0DecodeTest.java:95-126)."""
import json
import os

import numpy as np
import pytest

from oracle import pyoracle as O

HERE = os.path.dirname(os.path.abspath(__file__))
GOLDEN = os.path.join(HERE, "golden", "projection_golden.npz")
KNOWN = os.path.join(HERE, "golden", "reference_known_answers.json")
TYPES = {"q8_0": O.Q8_0, "q4_0": O.Q4_0, "q4_k": O.Q4_K}
N, D = 512, 37


@pytest.fixture(scope="module")
def gold():
    return np.load(GOLDEN)


def bits(a):
    return np.ascontiguousarray(a, dtype=np.float32).view(np.uint32)


def test_reference_known_answers():
    k = json.load(open(KNOWN))
    q = k["q4_0_decode"]
    raw = np.zeros(q["block_bytes_total"], dtype=np.uint8)
    for i, v in q["block_bytes_nonzero"].items():
        raw[int(i)] = v
    for i, want in q["expected"].items():
        assert O.get_float(O.Q4_0, raw, int(i)) == want
    r = O.JavaRandom(42)
    assert [r.next_int(10) for _ in range(5)] == k["java_util_random"]["seed_42_next_int_10"]


@pytest.mark.parametrize("name", list(TYPES))
def test_oracle_reproduces_golden(gold, name):
    t = TYPES[name]
    x = gold["probe_x"]
    raw = gold[f"{name}.probe.raw"]
    head = raw[: gold[f"{name}.probe.dequant"].size // O.block_elems(t) * O.block_bytes(t)]
    assert np.array_equal(bits(O.dequant(t, head)), bits(gold[f"{name}.probe.dequant"]))
    assert np.array_equal(bits(O.matmul(t, raw, x, D, N, O.DOT_SCALAR)), bits(gold[f"{name}.probe.matvec_scalar"]))
    assert np.array_equal(bits(O.matmul(t, raw, x, D, N, O.DOT_VEC256)), bits(gold[f"{name}.probe.matvec_vec256"]))
    assert np.array_equal(bits(O.dequant(t, gold[f"{name}.adversarial.raw"])), bits(gold[f"{name}.adversarial.dequant"]))
    got = O.matmul_batch(t, gold[f"{name}.batch.raw"], gold[f"{name}.batch.X"], D, N)
    assert np.array_equal(bits(got), bits(gold[f"{name}.batch.out"]))
    w1, w3, xs = gold[f"{name}.gate_up.w1"], gold[f"{name}.gate_up.w3"], gold[f"{name}.gate_up.x"]
    d = gold[f"{name}.gate_up.out"].size
    g = O.matmul(t, w1, xs, d, xs.size, O.DOT_SCALAR)
    u = O.matmul(t, w3, xs, d, xs.size, O.DOT_SCALAR)
    assert np.array_equal(bits(O.swiglu(g, u)), bits(gold[f"{name}.gate_up.out"]))


# ---- GPU: the library against the committed values -------------------------------------------

@pytest.fixture(scope="module")
def ctx():
    from jitllm_amd.runtime import Context
    c = Context(0)
    yield c
    c.close()


def magnitude(w, X, rows, cols):
    """sum_j |w_ij x_j| from decoded weights (float64)."""
    return np.abs(w.reshape(rows, cols).astype(np.float64)) @ np.abs(np.atleast_2d(X).astype(np.float64)).T


@pytest.mark.gpu
@pytest.mark.parametrize("name", list(TYPES))
def test_hip_matches_golden(ctx, gold, name):
    from gpu_util import say
    from jitllm_amd.projections import QuantizedBatchProjections, QuantizedProjections, TornadoWorkspace
    t = TYPES[name]
    say("golden", name)
    # element decode: bit for bit, adversarial scales included
    adv = gold[f"{name}.adversarial.raw"]
    cols = 256
    rows = adv.size // O.block_bytes(t) * O.block_elems(t) // cols
    w = ctx.load_weight(t, adv, rows, cols)
    assert np.array_equal(bits(w.dequantize().reshape(-1)), bits(gold[f"{name}.adversarial.dequant"]))
    # single-vector projection on the reference's probe fixture
    raw, x = gold[f"{name}.probe.raw"], gold["probe_x"]
    wp = ctx.load_weight(t, raw, D, N)
    dec = wp.dequantize()
    mag = magnitude(dec, x, D, N)[:, 0]
    proj = QuantizedProjections(ctx, TornadoWorkspace(wrapXb=ctx.from_numpy(x)))
    out = ctx.float_array(D)
    proj.matvec(out, wp, N, D)
    ctx.sync()
    want = gold[f"{name}.probe.matvec_scalar"]
    got = out.get()
    assert np.max(np.abs(got - want) / np.maximum(mag, 1e-30)) < 1e-3
    assert np.all(np.abs(got - want) <= np.maximum(1e-3, 1e-4 * np.abs(want)))  # the reference test's own tolerance
    # batched rows (fp16 MFMA path: 2e-3 of the magnitude)
    braw, X = gold[f"{name}.batch.raw"], gold[f"{name}.batch.X"]
    wb = ctx.load_weight(t, braw, D, N)
    bmag = magnitude(wb.dequantize(), X, D, N).T
    bout = ctx.float_array(X.shape[0] * D)
    QuantizedBatchProjections(ctx, X.shape[0], N, D).projection(ctx.from_numpy(X), bout, wb, N, D, False)
    ctx.sync()
    err = np.abs(bout.get().reshape(X.shape[0], D) - gold[f"{name}.batch.out"]) / np.maximum(bmag, 1e-30)
    assert err.max() < 2e-3
    # fused gate/up with SwiGLU
    w1, w3, xs = gold[f"{name}.gate_up.w1"], gold[f"{name}.gate_up.w3"], gold[f"{name}.gate_up.x"]
    d = gold[f"{name}.gate_up.out"].size
    h1, h3 = ctx.load_weight(t, w1, d, xs.size), ctx.load_weight(t, w3, d, xs.size)
    ws = TornadoWorkspace(wrapXb=ctx.from_numpy(xs), wrapHb=ctx.float_array(d))
    QuantizedProjections(ctx, ws).gateUp(h1, h3, xs.size, d)
    ctx.sync()
    want = gold[f"{name}.gate_up.out"]
    got = ws.wrapHb.get()
    scale = np.abs(want).max()
    assert np.max(np.abs(got - want)) < 1e-3 * max(scale, 1.0)
