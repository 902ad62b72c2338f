"""GPU parity at the full sizes of the benchmark's configurations.

The HIP path runs the whole shape; the oracle checks a sample of it -- a few hundred weight rows
gathered into a small matrix (rows are independent dot products, FloatTensor.java:123-125), and for
the batched calls a few dozen activation rows -- so that every launch geometry the benchmark times
has an oracle comparison without minutes of scalar CPU work.  The sample always holds the first and
the last rows (tile edges) and a seeded random remainder.
"""
import numpy as np
import pytest

from gpu_util import magnitude, rel_err, say
from oracle import pyoracle as O

pytestmark = pytest.mark.gpu

NAMES = {O.Q8_0: "q8_0", O.Q4_0: "q4_0", O.Q4_K: "q4_K"}
BLOCK = {O.Q8_0: (32, 34), O.Q4_0: (32, 18), O.Q4_K: (256, 144)}
POISON = np.float32(-999999.0)


@pytest.fixture(scope="module")
def ctx():
    from jitllm_amd.runtime import Context
    c = Context(0)
    yield c
    c.close()


def row_bytes(t, n):
    elems, nbytes = BLOCK[t]
    return n // elems * nbytes


def sample_rows(d, count, seed):
    """Sorted row indices: the first 16, the last 16 and a random remainder."""
    rng = np.random.default_rng(seed)
    edge = np.concatenate([np.arange(min(16, d)), np.arange(max(0, d - 16), d)])
    rest = rng.choice(d, size=min(count, d), replace=False)
    return np.unique(np.concatenate([edge, rest]))


def gather(raw, t, n, rows):
    return np.ascontiguousarray(raw.reshape(-1, row_bytes(t, n))[rows]).reshape(-1)


def dot_mode(t):
    return O.DOT_SCALAR if t == O.Q4_K else O.DOT_VEC256


# ---- single-token projections (configurations 2 and 3) -----------------------------------------

def test_vocabulary_projection_128256(ctx):
    """Q8_0 128256 x 2048 through floatMatvec and through the RMS-folding form
    (LogitsQ8_0Layer.java:238-247), the largest launch of the decode set."""
    from jitllm_amd import synthetic
    from jitllm_amd.projections import QuantizedProjections, TornadoWorkspace
    t, d, n = O.Q8_0, 128256, 2048
    say("vocabulary projection", d, n)
    raw = synthetic.weight(t, d, n, seed=18)
    x = synthetic.activations(n, seed=901)
    rw = (1.0 + 0.25 * synthetic.activations(n, seed=902)).astype(np.float32)
    rows = sample_rows(d, 384, 903)
    sub = gather(raw, t, n, rows)
    w = ctx.load_weight(t, raw, d, n)
    proj = QuantizedProjections(ctx, TornadoWorkspace())
    dx, logits = ctx.from_numpy(x), ctx.float_array(d, fill=POISON)
    proj.floatMatvec(dx, logits, w, n, d)
    ctx.sync()
    got = logits.get()
    assert np.all(got != POISON)
    ref = O.matmul(t, sub, x, rows.size, n, O.DOT_VEC256)
    assert rel_err(got[rows], ref, magnitude(t, sub, x, rows.size, n)) < 2e-5
    xn = O.rmsnorm(x, rw, 1e-5)
    logits.init(POISON)
    proj.rmsMatvec(dx, ctx.from_numpy(rw), None, logits, w, n, d, eps=1e-5)
    ctx.sync()
    got = logits.get()
    assert np.all(got != POISON)
    ref = O.matmul(t, sub, xn, rows.size, n, O.DOT_VEC256)
    assert rel_err(got[rows], ref, magnitude(t, sub, xn, rows.size, n)) < 2e-5
    # the greedy token over all 128 256 logits
    token = ctx.raw_buffer(4)
    proj.argmax(logits, d, token)
    ctx.sync()
    assert int(token.download(np.int32, 1)[0]) == O.argmax(got)
    w.free()


@pytest.mark.parametrize("B", [64, 96, 128])
def test_vocabulary_projection_for_many_sequences(ctx, B):
    """The same 128256 x 2048 weight for B rows of activations: two and three row blocks of the
    weight-streaming kernel and, at 128 rows, the tiled kernel that decodes in its loop -- a call
    of 279 MB, where the streaming kernel is still the cheaper at 96 rows."""
    from jitllm_amd import synthetic
    from jitllm_amd.projections import QuantizedBatchProjections
    t, d, n = O.Q8_0, 128256, 2048
    say("vocabulary projection, rows", B)
    raw = synthetic.weight(t, d, n, seed=18)
    rows = sample_rows(d, 96, 905)
    sub = gather(raw, t, n, rows)
    w = ctx.load_weight(t, raw, d, n)
    del raw
    X = synthetic.activations((B, n), seed=906 + B)
    proj = QuantizedBatchProjections(ctx, B, n, d)
    out = ctx.float_array(B * d, fill=POISON)
    proj.projection(ctx.from_numpy(X), out, w, n, d, False)
    ctx.sync()
    got = out.get().reshape(B, d)
    assert np.all(got != POISON)
    ref = O.matmul_batch(t, sub, X, rows.size, n)
    assert rel_err(got[:, rows], ref, magnitude(t, sub, X, rows.size, n)) < 2e-3
    out.free()
    proj.workspace.free()
    w.free()


@pytest.mark.parametrize("d,n", [(4096, 14336), (14336, 4096)])
def test_q4_0_llama3_8b_feed_forward_shapes(ctx, d, n):
    """Q4_0 w2 4096 x 14336 (rows of 14336 columns) and w1 / w3 14336 x 4096, plain and residual."""
    from jitllm_amd import synthetic
    from jitllm_amd.projections import QuantizedProjections, TornadoWorkspace
    t = O.Q4_0
    say("q4_0 8B shape", d, n)
    raw = synthetic.weight(t, d, n, seed=910 + d % 7)
    x = synthetic.activations(n, seed=911)
    rows = sample_rows(d, 256, 912)
    sub = gather(raw, t, n, rows)
    ref = O.matmul(t, sub, x, rows.size, n, O.DOT_VEC256)
    mag = magnitude(t, sub, x, rows.size, n)
    w = ctx.load_weight(t, raw, d, n)
    base = synthetic.activations(d, seed=913)
    acc = ctx.from_numpy(base)
    proj = QuantizedProjections(ctx, TornadoWorkspace(wrapX=acc))
    out = ctx.float_array(d, fill=POISON)
    proj.floatMatvec(ctx.from_numpy(x), out, w, n, d)
    proj.residualMatvec(ctx.from_numpy(x), w, n, d)
    ctx.sync()
    got = out.get()
    assert np.all(got != POISON)
    assert rel_err(got[rows], ref, mag) < 2e-5
    assert rel_err(acc.get()[rows] - base[rows], ref, mag + np.abs(base[rows]) * 1e-6 + 1e-30) < 2e-5
    w.free()


# ---- Q4_K batched decode (configuration 4) -----------------------------------------------------

@pytest.mark.parametrize("B", [8, 32, 64])
def test_q4_k_batched_gate_up_12288(ctx, B):
    """hb = SiLU(w1 . x) * (w3 . x), 2 x [12288 x 4096] Q4_K, B sequences."""
    from jitllm_amd import synthetic
    from jitllm_amd.projections import QuantizedBatchProjections
    t, d, n = O.Q4_K, 12288, 4096
    say("q4_K batched gate/up", B)
    r1 = synthetic.weight(t, d, n, seed=65)
    r3 = synthetic.weight(t, d, n, seed=66)
    X = synthetic.activations((B, n), seed=920 + B)
    rows = sample_rows(d, 192, 921)
    s1, s3 = gather(r1, t, n, rows), gather(r3, t, n, rows)
    g = O.matmul_batch(t, s1, X, rows.size, n, O.DOT_SCALAR)
    u = O.matmul_batch(t, s3, X, rows.size, n, O.DOT_SCALAR)
    ref = O.swiglu(g.reshape(-1), u.reshape(-1)).reshape(B, rows.size)
    w1, w3 = ctx.load_weight(t, r1, d, n), ctx.load_weight(t, r3, d, n)
    hb = ctx.float_array(B * d, fill=POISON)
    QuantizedBatchProjections(ctx, B, n, 2 * d).gateUp(ctx.from_numpy(X), hb, w1, w3, n, d)
    ctx.sync()
    got = hb.get().reshape(B, d)
    assert np.all(got != POISON)
    mg, mu = magnitude(t, s1, X, rows.size, n), magnitude(t, s3, X, rows.size, n)
    bound = 2e-4 * (mg * np.abs(u) + 1.2 * mu * np.abs(g)) + 1e-6
    assert np.all(np.abs(got[:, rows].astype(np.float64) - ref) <= bound)
    w1.free()
    w3.free()


@pytest.mark.parametrize("B", [8, 32, 64])
def test_q4_k_batched_down_projection_12288(ctx, B):
    """The ffn-wide down projection 4096 x 12288 Q4_K with the residual add, B sequences."""
    from jitllm_amd import synthetic
    from jitllm_amd.projections import QuantizedBatchProjections
    t, d, n = O.Q4_K, 4096, 12288
    say("q4_K batched down", B)
    raw = synthetic.weight(t, d, n, seed=67)
    X = synthetic.activations((B, n), seed=930 + B) * np.float32(0.1)
    rows = sample_rows(d, 192, 931)
    sub = gather(raw, t, n, rows)
    ref = O.matmul_batch(t, sub, X, rows.size, n, O.DOT_SCALAR)
    mag = magnitude(t, sub, X, rows.size, n)
    w = ctx.load_weight(t, raw, d, n)
    base = synthetic.activations((B, d), seed=932)
    out = ctx.from_numpy(base)
    QuantizedBatchProjections(ctx, B, n, d).projection(ctx.from_numpy(X), out, w, n, d, True)
    ctx.sync()
    got = out.get().reshape(B, d)
    err = rel_err(got[:, rows] - base[:, rows], ref, mag + np.abs(base[:, rows]) * 1e-6)
    assert err < 2e-4, err
    w.free()


@pytest.mark.parametrize("B", [8, 32, 64])
def test_q4_k_batched_qkv_and_o(ctx, B):
    """q|k|v (4096 + 1024 + 1024 rows side by side) and o (4096 x 4096) of the Qwen3-8B-like layer."""
    from jitllm_amd import synthetic
    from jitllm_amd.projections import QuantizedBatchProjections
    t, n = O.Q4_K, 4096
    dims = (4096, 1024, 1024)
    say("q4_K batched qkv + o", B)
    raws = [synthetic.weight(t, d, n, seed=61 + i) for i, d in enumerate(dims)]
    X = synthetic.activations((B, n), seed=940 + B)
    ws = [ctx.load_weight(t, r, d, n) for r, d in zip(raws, dims)]
    ld = sum(dims)
    out = ctx.float_array(B * ld, fill=POISON)
    proj = QuantizedBatchProjections(ctx, B, n, ld)
    dX = ctx.from_numpy(X)
    proj.fusedQKV(dX, out, *ws)
    o = ctx.float_array(B * 4096, fill=POISON)
    proj.projection(dX, o, ws[0], n, 4096, False)
    ctx.sync()
    got = out.get().reshape(B, ld)
    assert np.all(got != POISON)
    col = 0
    for raw, d in zip(raws, dims):
        rows = sample_rows(d, 96, 941 + d)
        sub = gather(raw, t, n, rows)
        ref = O.matmul_batch(t, sub, X, rows.size, n, O.DOT_SCALAR)
        err = rel_err(got[:, col + rows], ref, magnitude(t, sub, X, rows.size, n))
        assert err < 2e-4, (d, err)
        if d == 4096:
            assert rel_err(o.get().reshape(B, d)[:, rows], ref, magnitude(t, sub, X, rows.size, n)) < 2e-4
        col += d
    for w in ws:
        w.free()


# ---- Q8_0 batched prefill (configuration 5, fp32 X through jl_gemm) ----------------------------

@pytest.mark.parametrize("T", [512, 2048])
def test_q8_0_prefill_down_projection_k8192(ctx, T):
    """out += X . W2^T with rows of 8192 columns (2048 x 8192 Q8_0), T tokens."""
    from jitllm_amd import synthetic
    from jitllm_amd.projections import QuantizedBatchProjections
    t, d, n = O.Q8_0, 2048, 8192
    say("prefill down", T)
    raw = synthetic.weight(t, d, n, seed=47)
    X = synthetic.activations((T, n), seed=950 + T) * np.float32(0.1)
    rows = sample_rows(d, 224, 951)
    toks = sample_rows(T, 16, 952)
    sub = gather(raw, t, n, rows)
    ref = O.matmul_batch(t, sub, X[toks], rows.size, n, O.DOT_VEC256)
    mag = magnitude(t, sub, X[toks], rows.size, n)
    w = ctx.load_weight(t, raw, d, n)
    base = synthetic.activations((T, d), seed=953)
    out = ctx.from_numpy(base)
    QuantizedBatchProjections(ctx, T, n, d).projection(ctx.from_numpy(X), out, w, n, d, True)
    ctx.sync()
    got = out.get().reshape(T, d)
    sel = got[np.ix_(toks, rows)] - base[np.ix_(toks, rows)]
    err = rel_err(sel, ref, mag + np.abs(base[np.ix_(toks, rows)]) * 1e-6)
    assert err < 2e-4, err
    w.free()


@pytest.mark.parametrize("T", [512, 2048])
def test_q8_0_prefill_gate_up_n16384(ctx, T):
    """hb = SiLU(X . W1^T) * (X . W3^T), 2 x [8192 x 2048] Q8_0 (16 384 output columns), T tokens."""
    from jitllm_amd import synthetic
    from jitllm_amd.projections import QuantizedBatchProjections
    t, d, n = O.Q8_0, 8192, 2048
    say("prefill gate/up", T)
    r1 = synthetic.weight(t, d, n, seed=45)
    r3 = synthetic.weight(t, d, n, seed=46)
    X = synthetic.activations((T, n), seed=960 + T)
    rows = sample_rows(d, 224, 961)
    toks = sample_rows(T, 16, 962)
    s1, s3 = gather(r1, t, n, rows), gather(r3, t, n, rows)
    g = O.matmul_batch(t, s1, X[toks], rows.size, n, O.DOT_VEC256)
    u = O.matmul_batch(t, s3, X[toks], rows.size, n, O.DOT_VEC256)
    ref = O.swiglu(g.reshape(-1), u.reshape(-1)).reshape(toks.size, rows.size)
    w1, w3 = ctx.load_weight(t, r1, d, n), ctx.load_weight(t, r3, d, n)
    hb = ctx.float_array(T * d, fill=POISON)
    QuantizedBatchProjections(ctx, T, n, 2 * d).gateUp(ctx.from_numpy(X), hb, w1, w3, n, d)
    ctx.sync()
    got = hb.get().reshape(T, d)
    assert np.all(got != POISON)
    mg, mu = magnitude(t, s1, X[toks], rows.size, n), magnitude(t, s3, X[toks], rows.size, n)
    bound = 2e-4 * (mg * np.abs(u) + 1.2 * mu * np.abs(g)) + 1e-6
    assert np.all(np.abs(got[np.ix_(toks, rows)].astype(np.float64) - ref) <= bound)
    w1.free()
    w3.free()


@pytest.mark.parametrize("T", [512, 2048])
def test_q8_0_prefill_qkv_and_o(ctx, T):
    """q|k|v (2048 + 512 + 512 side by side) and o (2048 x 2048, residual) at the benchmark's T."""
    from jitllm_amd import synthetic
    from jitllm_amd.projections import QuantizedBatchProjections
    t, n = O.Q8_0, 2048
    dims = (2048, 512, 512)
    say("prefill qkv + o", T)
    raws = [synthetic.weight(t, d, n, seed=41 + i) for i, d in enumerate(dims)]
    X = synthetic.activations((T, n), seed=970 + T)
    toks = sample_rows(T, 16, 971)
    ws = [ctx.load_weight(t, r, d, n) for r, d in zip(raws, dims)]
    ld = sum(dims)
    out = ctx.float_array(T * ld, fill=POISON)
    proj = QuantizedBatchProjections(ctx, T, n, ld)
    dX = ctx.from_numpy(X)
    proj.fusedQKV(dX, out, *ws)
    base = synthetic.activations((T, 2048), seed=972)
    acc = ctx.from_numpy(base)
    proj.projection(dX, acc, ws[0], n, 2048, True)
    ctx.sync()
    got = out.get().reshape(T, ld)
    assert np.all(got != POISON)
    col = 0
    for raw, d in zip(raws, dims):
        rows = sample_rows(d, 96, 973 + d)
        sub = gather(raw, t, n, rows)
        ref = O.matmul_batch(t, sub, X[toks], rows.size, n, O.DOT_VEC256)
        mag = magnitude(t, sub, X[toks], rows.size, n)
        assert rel_err(got[np.ix_(toks, col + rows)], ref, mag) < 2e-4
        if d == 2048:
            sel = acc.get().reshape(T, d)[np.ix_(toks, rows)] - base[np.ix_(toks, rows)]
            assert rel_err(sel, ref, mag + np.abs(base[np.ix_(toks, rows)]) * 1e-6) < 2e-4
        col += d
    for w in ws:
        w.free()


# ---- a weight past 2 GiB ---------------------------------------------------------------------------

def test_a_weight_of_more_than_two_gib(ctx):
    """Q8_0 140000 x 16384 is 2.44e9 bytes: byte offsets into it do not fit 32 bits.  The single-token
    projection, batched decode (8 and 40 rows), a mid row count (200) and prefill (600 rows, a 4.9 GB
    fp16 copy in the workspace) over it, held to the oracle on the first and last rows, a random
    sample and the rows on either side of the 2^31-byte mark; every output is written."""
    from jitllm_amd import synthetic
    from jitllm_amd.projections import QuantizedBatchProjections, QuantizedProjections, TornadoWorkspace
    t, d, n = O.Q8_0, 140000, 16384
    say("a weight past 2 GiB", d, n)
    part = synthetic.weight(t, 20000, n, seed=31)
    rb = row_bytes(t, n)
    raw = np.concatenate([np.roll(part.reshape(20000, rb), i, axis=0).reshape(-1) for i in range(7)])
    assert raw.size > 2 ** 31
    mark = 2 ** 31 // rb
    rows = np.unique(np.concatenate([sample_rows(d, 64, 32), np.arange(mark - 4, mark + 4)]))
    sub = gather(raw, t, n, rows)
    w = ctx.load_weight(t, raw, d, n)
    del raw
    x = synthetic.activations(n, seed=33)
    out = ctx.float_array(d, fill=POISON)
    QuantizedProjections(ctx, TornadoWorkspace()).floatMatvec(ctx.from_numpy(x), out, w, n, d)
    ctx.sync()
    got = out.get()
    assert np.all(got != POISON)
    assert rel_err(got[rows], O.matmul(t, sub, x, rows.size, n), magnitude(t, sub, x, rows.size, n)) < 2e-5
    out.free()
    for B in (8, 40, 200, 600):
        say("a weight past 2 GiB, rows", B)
        X = synthetic.activations((B, n), seed=34 + B)
        proj = QuantizedBatchProjections(ctx, B, n, d)
        o = ctx.float_array(B * d, fill=POISON)
        proj.projection(ctx.from_numpy(X), o, w, n, d, False)
        ctx.sync()
        g = o.get().reshape(B, d)
        assert np.all(g != POISON)
        assert rel_err(g[:, rows], O.matmul_batch(t, sub, X, rows.size, n), magnitude(t, sub, X, rows.size, n)) < 2e-3
        o.free()
        proj.workspace.free()
    w.free()
