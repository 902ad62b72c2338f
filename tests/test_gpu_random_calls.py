"""Seeded random calls across the entry points: every weight type, row lengths and row counts on
both sides of every dispatch threshold, partial batches, row strides and column offsets, pointers
that start off a 16-byte boundary, fp32 and binary16 activations, kept fp16 copies, workspaces of
the least size a call accepts.  The reference is a float64 product of the weights as the numpy
models decode them (the int8 mode: the oracle's statement of its arithmetic, bit for bit); a call
the library refuses must leave its outputs alone.  Two bugs of shape dispatch were found this way
(a fused q|k|v whose first weight was the shortest, a kept copy whose partial sums had no room in
the workspace): both are kept below as cases of their own."""
import numpy as np
import pytest

import np_models as NP
from gpu_util import say
from oracle import pyoracle as O

pytestmark = pytest.mark.gpu

UNTOUCHED = np.float32(-12345.5)
GUARD = np.float32(-999999.0)
MAIN = [O.Q8_0, O.Q4_0, O.Q4_K]
MINOR = [O.Q5_K, O.Q6_K, O.Q4_1, O.Q5_0, O.IQ4_XS]
BLOCK = {O.Q8_0: 32, O.Q4_0: 32, O.Q4_1: 32, O.Q5_0: 32, O.Q4_K: 256, O.Q5_K: 256, O.Q6_K: 256, O.IQ4_XS: 256}
ROW_LENGTHS = [256, 512, 768, 1024, 1536, 2048, 2304, 2560, 3072, 3584, 4096, 5120, 6144, 8192, 11008, 12288, 14336]
F16_BOUND = 2e-3     # fp16-MFMA paths: |d| / sum |w x|
F32_BOUND = 2e-5     # fp32 paths


@pytest.fixture(scope="module")
def ctx():
    from jitllm_amd.runtime import Context
    c = Context(0)
    yield c
    c.close()


class Shifted:
    """An fp32 device array that starts ``shift`` floats into its allocation, guard floats on both sides."""

    def __init__(self, ctx, values, shift):
        values = np.ascontiguousarray(values, dtype=np.float32).reshape(-1)
        self.buf = ctx.float_array(values.size + shift + 4, fill=float(GUARD))
        self.shift, self.size = shift, values.size
        self.buf.upload(values, offset=4 * shift)
        self.ptr = self.buf.ptr.value + 4 * shift

    def get(self):
        whole = self.buf.download(np.float32, self.size + self.shift + 4)
        guards = np.concatenate([whole[:self.shift], whole[self.shift + self.size:]])
        assert np.all(guards == GUARD), "a call wrote outside its output"
        return whole[self.shift:self.shift + self.size]

    def free(self):
        self.buf.free()


def decoded(t, raw, d, n):
    return NP.DEQUANT[t](raw).reshape(d, n).astype(np.float64)


def silu_times(g, u):
    return g / (1.0 + np.exp(-g)) * u


# ---- batched calls: jl_gemm / jl_gemm_resident / jl_gemm_xf16 -------------------------------------

def batched_case(rng):
    t = int(rng.choice(MAIN if rng.random() < 0.7 else MINOR))
    n = int(rng.choice(ROW_LENGTHS))
    r = rng.random()
    batch = (int(rng.integers(1, 65)) if r < 0.25 else int(rng.integers(65, 512)) if r < 0.55 else
             int(rng.integers(512, 1100)) if r < 0.8 else
             int(rng.choice([8, 16, 32, 64, 128, 192, 256, 384, 511, 512, 513, 1024, 2048])))
    active = batch if rng.random() < 0.6 else int(rng.integers(1, batch + 1))
    form = str(rng.choice(["one", "side", "swiglu"], p=[0.5, 0.25, 0.25]))
    budget = max(1, (16_000_000 if batch <= 600 else 8_000_000) // n)

    def width(limit):
        r = rng.random()
        d = (int(rng.integers(1, 600)) if r < 0.3 else int(rng.integers(600, 4200)) if r < 0.6 else
             int(rng.choice([128, 256, 512, 1024, 2048, 4096, 6144, 8192, 12288, 16384])) if r < 0.8 else
             int(rng.integers(4200, 17000)))
        return max(1, min(d, limit))

    if form == "one":
        dims = [width(budget)]
    elif form == "side":
        k = int(rng.integers(2, 4))
        dims = [width(budget // k) for _ in range(k)]
    else:
        dims = [width(budget // 2)] * 2
    swiglu = form == "swiglu"
    residual = (not swiglu) and rng.random() < 0.4
    total = dims[0] if swiglu else sum(dims)
    col_offset = int(rng.choice([0, 0, 0, 3, 64, 100]))
    ldo = col_offset + total + int(rng.choice([0, 0, 5, 128]))
    xf16 = rng.random() < 0.4
    c_f16 = bool(xf16 and swiglu and rng.random() < 0.5)
    resident = rng.random() < 0.4
    tight = bool(resident and rng.random() < 0.3)
    shift = int(rng.choice([0, 0, 0, 1, 2, 3]))
    # one call in six with more than one weight mixes types (each weight is then decoded by its own)
    types = [t] * len(dims)
    if len(dims) > 1 and rng.random() < 0.35:
        types = [int(rng.choice(MAIN + MINOR)) for _ in dims]
    return dict(t=t, types=types, n=n, batch=batch, active=active, dims=dims, swiglu=swiglu, residual=residual, col_offset=col_offset,
                ldo=ldo, xf16=xf16, c_f16=c_f16, resident=resident, tight=tight, shift=shift)


def run_batched_case(ctx, c, seed):
    from jitllm_amd import _lib as L, synthetic
    from jitllm_amd.projections import QuantizedBatchProjections
    t, n, batch, active, dims, ldo, col_offset = c["t"], c["n"], c["batch"], c["active"], c["dims"], c["ldo"], c["col_offset"]
    swiglu, residual, c_f16 = c["swiglu"], c["residual"], c["c_f16"]
    total = dims[0] if swiglu else sum(dims)
    types = c.get("types", [t] * len(dims))
    raws = [synthetic.weight(ti, d, n, seed=seed + i) for i, (ti, d) in enumerate(zip(types, dims))]
    ws = [ctx.load_weight(ti, r, d, n) for ti, r, d in zip(types, raws, dims)]
    X = synthetic.activations((batch, n), seed=seed + 7)
    if c["xf16"]:
        X16 = X.astype(np.float16)
        X = X16.astype(np.float32)
    if c_f16:
        start = np.full((batch, ldo), 7.5, dtype=np.float16)
    elif residual:
        start = synthetic.activations((batch, ldo), seed=seed + 8)
    else:
        start = np.full((batch, ldo), UNTOUCHED, dtype=np.float32)
    # (a kept copy needs no room in the workspace: `tight` brings the activations' region only)
    proj = QuantizedBatchProjections(ctx, batch, n, 0 if c["tight"] else sum(dims), resident=c["resident"])
    epilogue = L.JL_SWIGLU if swiglu else L.JL_RESIDUAL if residual else L.JL_STORE
    outs = []
    for _ in range(2):
        out = ctx.half_from_numpy(start.reshape(-1)) if c_f16 else Shifted(ctx, start, c["shift"])
        x = ctx.half_from_numpy(X16.reshape(-1)) if c["xf16"] else ctx.from_numpy(X.reshape(-1))
        proj._gemm(ws, x, out, active, ldo, col_offset, epilogue)
        outs.append(out)
    ctx.sync()
    a, b = (o.get().reshape(batch, ldo) for o in outs)
    bits = np.uint16 if c_f16 else np.uint32
    assert np.array_equal(a.view(bits), b.view(bits)), "the second call gives other bits"
    outside = np.ones((batch, ldo), dtype=bool)
    outside[:active, col_offset:col_offset + total] = False
    assert np.array_equal(a.view(bits)[outside], start.view(bits)[outside]), "wrote outside its rows and columns"
    Xa = X[:active].astype(np.float64)
    W = [decoded(ti, r, d, n) for ti, r, d in zip(types, raws, dims)]
    prods = [Xa @ w.T for w in W]
    mags = [np.abs(Xa) @ np.abs(w).T for w in W]
    got = a[:active, col_offset:col_offset + total].astype(np.float64)
    if swiglu:
        g, u = prods
        want = silu_times(g, u)
        bound = F16_BOUND * (mags[0] * np.abs(u) + 1.2 * mags[1] * np.abs(g)) + 1e-6
        if c_f16:
            bound = bound + np.abs(want) * 2.0 ** -11 + 2.0 ** -24
            in_range = np.abs(want) + bound < 65000.0       # beyond what binary16 holds infinity is the right answer
            got, want = np.where(in_range, got, 0.0), np.where(in_range, want, 0.0)
    else:
        want = np.concatenate(prods, axis=1)
        bound = F16_BOUND * np.concatenate(mags, axis=1)
        if residual:
            base = start[:active, col_offset:col_offset + total].astype(np.float64)
            want = want + base
            bound = bound + (np.abs(base) + np.abs(want)) * 2.0 ** -23
    assert np.all(np.isfinite(got))
    excess = np.abs(got - want) - bound
    assert excess.max() <= 0, (float(excess.max()), np.unravel_index(np.argmax(excess), excess.shape))
    for w in ws:
        w.free()
    for o in outs:
        o.free()
    proj.workspace.free()
    for copy in proj._copies.buffers():
        copy.free()


@pytest.mark.parametrize("chunk", range(8))
def test_random_batched_calls(ctx, chunk):
    rng = np.random.default_rng(20261100 + chunk)
    for i in range(24):
        c = batched_case(rng)
        if c["batch"] * c["ldo"] > 30_000_000:
            continue
        say("random batched call", chunk, i, c)
        run_batched_case(ctx, c, seed=(chunk * 100 + i) * 16 + 5000)


def test_found_by_random_calls_kept_copy_with_the_least_workspace(ctx):
    """Q6_K, 243 rows over a kept copy: the cheapest tiling cuts K, the partial sums need 12 MB and
    the workspace of a 243-row caller held 9.7 -- the call was refused; it now keeps K whole when
    there is no room (and the size query counts the partial sums from 128 rows)."""
    for tight in (False, True):
        c = dict(t=O.Q6_K, n=768, batch=243, active=243, dims=[5870], swiglu=False, residual=False, col_offset=64,
                 ldo=5934, xf16=False, c_f16=False, resident=True, tight=tight, shift=0)
        say("kept copy, least workspace", c)
        run_batched_case(ctx, c, seed=77)


# ---- single-token calls: every jl_gemv* entry point -----------------------------------------------

SINGLE_OPS = ["store", "residual", "qkv", "gate_up", "rms", "rms_residual", "qkv_rms", "gate_up_rms", "argmax",
              "argmax_rms", "q8", "q8_residual", "qkv_q8", "gate_up_q8"]


def single_case(rng):
    # (the fused and packed forms exist for the three main types: most cases go where there is a kernel)
    op = str(rng.choice(SINGLE_OPS))
    plain = op in ("store", "residual", "gate_up", "argmax")
    t = int(rng.choice(MAIN if (not plain or rng.random() < 0.5) else MINOR))
    b = BLOCK[t]
    r = rng.random()
    n = (int(rng.choice(ROW_LENGTHS + [16384])) if r < 0.6 else b * int(rng.integers(1, 16384 // b + 1)) if r < 0.8 else
         b * int(rng.integers(1, 3000 // b + 2)))
    budget = max(1, 24_000_000 // n)

    def rows(limit):
        r = rng.random()
        d = (int(rng.integers(1, 300)) if r < 0.3 else int(rng.integers(300, 5000)) if r < 0.6 else
             int(rng.choice([256, 512, 1024, 2048, 4096, 8192, 14336, 32000])) if r < 0.8 else int(rng.integers(5000, 40000)))
        return max(1, min(d, limit))

    if op.startswith("qkv"):
        dims = [rows(budget // 3) for _ in range(3)]
        if rng.random() < 0.5:
            dims[2] = dims[1]
    elif op.startswith("gate_up"):
        dims = [rows(budget // 2)] * 2
    else:
        dims = [rows(budget)]
    return dict(t=t, op=op, n=n, dims=dims, given_scale=bool(rng.random() < 0.5), eps=float(rng.choice([1e-5, 1e-6])),
                x_shift=int(rng.choice([0, 0, 0, 0, 1, 2, 4])), out_shift=int(rng.choice([0, 0, 0, 1, 2, 3, 4])))


def run_single_case(ctx, c, seed):
    """Returns False when the library refused the call (outputs checked untouched)."""
    from jitllm_amd import _lib as L, synthetic
    lib, h = L.load(), ctx.handle
    t, op, n, dims, eps = c["t"], c["op"], c["n"], c["dims"], c["eps"]
    raws = [synthetic.weight(t, d, n, seed=seed + i) for i, d in enumerate(dims)]
    ws = [ctx.load_weight(t, r, d, n) for r, d in zip(raws, dims)]
    x = synthetic.activations(n, seed=seed + 7)
    rw = (1.0 + 0.1 * synthetic.activations(n, seed=seed + 8)).astype(np.float32)
    dx, drw = Shifted(ctx, x, c["x_shift"]), ctx.from_numpy(rw)
    starts = [synthetic.activations(d, seed=seed + 9) if "residual" in op else np.full(d, GUARD, np.float32) for d in dims]
    nout = 1 if op.startswith("gate_up") else len(dims)
    outs = [Shifted(ctx, starts[i], c["out_shift"]) for i in range(nout)]
    scale, token = ctx.float_array(1, fill=0.0), ctx.raw_buffer(4)
    held = [dx, drw, scale, token] + outs
    xeff = x.astype(np.float64)
    scale_ptr = None
    st = 0
    if "rms" in op:
        ss = np.float32(1.0 / np.sqrt(np.sum(x.astype(np.float64) ** 2) / n + eps))
        xeff = rw.astype(np.float64) * (float(ss) * x.astype(np.float64))
        if c["given_scale"] and op != "gate_up_rms":
            L.check(lib.jl_rms_scale(h, dx.ptr, n, eps, scale.ptr))
            scale_ptr = scale.ptr
    if "q8" in op:
        dq, dsc, dsum = ctx.raw_buffer(max(n, 16)), ctx.float_array(n // 32), ctx.raw_buffer(max(n // 32 * 4, 16))
        held += [dq, dsc, dsum]
        st = lib.jl_quantize_q8(h, dx.ptr, n, dq.ptr, dsc.ptr, dsum.ptr)
        if st == 0:
            ctx.sync()
            xeff = dq.download(np.int8, n).astype(np.float64) * np.repeat(dsc.get().astype(np.float64), 32)
    w = [x_.handle for x_ in ws]
    o = [x_.ptr for x_ in outs]
    if st == 0:
        if op in ("store", "residual"):
            st = lib.jl_gemv(h, w[0], dx.ptr, o[0], L.JL_RESIDUAL if op == "residual" else L.JL_STORE)
        elif op == "qkv":
            st = lib.jl_gemv_qkv(h, *w, dx.ptr, *o)
        elif op == "gate_up":
            st = lib.jl_gemv_gate_up(h, *w, dx.ptr, o[0])
        elif op in ("rms", "rms_residual"):
            st = lib.jl_gemv_rms(h, w[0], dx.ptr, drw.ptr, scale_ptr, eps, o[0],
                                 L.JL_RESIDUAL if op == "rms_residual" else L.JL_STORE)
        elif op == "qkv_rms":
            st = lib.jl_gemv_qkv_rms(h, *w, dx.ptr, drw.ptr, scale_ptr, eps, *o)
        elif op == "gate_up_rms":
            st = lib.jl_gemv_gate_up_rms(h, *w, dx.ptr, drw.ptr, eps, o[0])
        elif op == "argmax":
            st = lib.jl_gemv_argmax(h, w[0], dx.ptr, None, None, 0.0, o[0], token.ptr)
        elif op == "argmax_rms":
            st = lib.jl_gemv_argmax(h, w[0], dx.ptr, drw.ptr, scale_ptr, eps, o[0], token.ptr)
        elif op in ("q8", "q8_residual"):
            st = lib.jl_gemv_q8(h, w[0], dq.ptr, dsc.ptr, dsum.ptr, o[0], L.JL_RESIDUAL if op == "q8_residual" else L.JL_STORE)
        elif op == "qkv_q8":
            st = lib.jl_gemv_qkv_q8(h, *w, dq.ptr, dsc.ptr, dsum.ptr, *o)
        else:
            st = lib.jl_gemv_gate_up_q8(h, *w, dq.ptr, dsc.ptr, dsum.ptr, o[0])
    ctx.sync()
    taken = st == 0
    if st == L.JL_ERR_UNSUPPORTED:
        # refused by name; nothing was launched
        assert lib.jl_last_error()
        for i in range(nout):
            assert np.array_equal(outs[i].get().view(np.uint32), starts[i].view(np.uint32))
    else:
        assert st == 0, (st, lib.jl_last_error())
        W = [decoded(t, r, d, n) for r, d in zip(raws, dims)]
        prods = [m @ xeff for m in W]
        mags = [np.abs(m) @ np.abs(xeff) for m in W]
        if op.startswith("gate_up"):
            g, u = prods
            want = [silu_times(g, u)]
            bounds = [F32_BOUND * (mags[0] * np.abs(u) + 1.2 * mags[1] * np.abs(g)) + 1e-6]
        else:
            want, bounds = prods, [F32_BOUND * m + 1e-30 for m in mags]
        for i in range(nout):
            got = outs[i].get().astype(np.float64)
            w_i, b_i = want[i], bounds[i]
            if "residual" in op:
                w_i = w_i + starts[i]
                b_i = b_i + (np.abs(starts[i]) + np.abs(w_i)) * 2.0 ** -23
            assert np.all(np.isfinite(got))
            excess = np.abs(got - w_i) - b_i
            assert excess.max() <= 0, (i, float(excess.max()), int(np.argmax(excess)))
        if op.startswith("argmax"):
            assert int(token.download(np.int32, 1)[0]) == int(np.argmax(outs[0].get()))
    for x_ in ws + held:
        x_.free()
    return taken


@pytest.mark.parametrize("chunk", range(8))
def test_random_single_token_calls(ctx, chunk):
    rng = np.random.default_rng(20261200 + chunk)
    taken = 0
    for i in range(40):
        c = single_case(rng)
        say("random single-token call", chunk, i, c)
        taken += run_single_case(ctx, c, seed=(chunk * 100 + i) * 16 + 9000)
    assert taken >= 20     # most cases are ones the library has a kernel for


def test_found_by_random_calls_fused_qkv_with_a_short_first_weight(ctx):
    """Q8_0 rows of 3008 columns (47 of 64 slices) and a q of 276 rows beside k / v of 1024: the
    fixed-geometry kernel measured every weight's tiles against the first weight's row count and
    read k and v past that point from the wrong place."""
    for t, n, dims in ((O.Q8_0, 3008, [276, 1024, 1024]), (O.Q4_0, 6144, [198, 242, 242])):
        c = dict(t=t, op="qkv", n=n, dims=dims, given_scale=False, eps=1e-5, x_shift=0, out_shift=0)
        say("qkv, short first weight", c)
        assert run_single_case(ctx, c, seed=4242)


# ---- the int8 mode ----------------------------------------------------------------------------------

@pytest.mark.parametrize("chunk", range(4))
def test_random_int8_calls(ctx, chunk):
    """jl_gemm with JL_MATH_INT8 at random shapes: plain, residual and side-by-side calls equal the
    oracle's block-scaled int8 arithmetic bit for bit; gate/up is SiLU(gate) * up of two such results."""
    from jitllm_amd import _lib as L, synthetic
    from jitllm_amd.projections import QuantizedBatchProjections
    rng = np.random.default_rng(20261300 + chunk)
    for i in range(30):
        t = int(rng.choice([O.Q8_0, O.Q4_0]))
        n = 64 * int(rng.choice([1, 2, 3, 4, 5, 8, 16, 24, 32, 48, 64, 128]))
        batch = int(rng.choice([int(rng.integers(1, 65)), int(rng.integers(65, 400)), int(rng.integers(400, 1100))]))
        active = batch if rng.random() < 0.6 else int(rng.integers(1, batch + 1))
        form = str(rng.choice(["one", "side", "swiglu"], p=[0.5, 0.3, 0.2]))
        budget = max(1, int(4e8 // (n * active)))

        def width():
            d = int(rng.choice([int(rng.integers(1, 300)), int(rng.integers(300, 3000)),
                                int(rng.choice([128, 256, 512, 1024, 2048, 4096, 8192]))]))
            return max(1, min(d, budget))

        dims = [width()] if form == "one" else [width() for _ in range(int(rng.integers(2, 4)))] if form == "side" else [width()] * 2
        swiglu = form == "swiglu"
        residual = (not swiglu) and rng.random() < 0.4
        total = dims[0] if swiglu else sum(dims)
        col_offset = int(rng.choice([0, 0, 3, 64]))
        ldo = col_offset + total + int(rng.choice([0, 0, 5, 128]))
        say("random int8 call", chunk, i, t, n, dims, batch, active, form, residual, col_offset, ldo)
        seed = (chunk * 100 + i) * 16 + 13000
        raws = [synthetic.weight(t, d, n, seed=seed + j) for j, d in enumerate(dims)]
        ws = [ctx.load_weight(t, r, d, n) for r, d in zip(raws, dims)]
        X = synthetic.activations((batch, n), seed=seed + 7)
        start = synthetic.activations((batch, ldo), seed=seed + 8) if residual else np.full((batch, ldo), UNTOUCHED, np.float32)
        proj = QuantizedBatchProjections(ctx, batch, n, sum(dims), math=L.JL_MATH_INT8)
        out = ctx.from_numpy(start.reshape(-1))
        proj._gemm(ws, ctx.from_numpy(X.reshape(-1)), out, active, ldo, col_offset,
                   L.JL_SWIGLU if swiglu else L.JL_RESIDUAL if residual else L.JL_STORE)
        ctx.sync()
        a = out.get().reshape(batch, ldo)
        outside = np.ones((batch, ldo), dtype=bool)
        outside[:active, col_offset:col_offset + total] = False
        assert np.array_equal(a.view(np.uint32)[outside], start.view(np.uint32)[outside])
        aq, ascale = O.quantize_q8(X[:active])
        refs = [O.gemm_int8_block_scaled(t, aq, ascale, r, d) for r, d in zip(raws, dims)]
        got = a[:active, col_offset:col_offset + total]
        if swiglu:
            g, u = refs[0].astype(np.float64), refs[1].astype(np.float64)
            want = silu_times(g, u)
            assert np.all(np.abs(got - want) <= 4e-6 * (np.abs(want) + 1e-3 * np.abs(u)) + 1e-30)
        else:
            want = np.concatenate(refs, axis=1)
            if residual:
                want = start[:active, col_offset:col_offset + total] + want
            assert np.array_equal(got.view(np.uint32), np.ascontiguousarray(want, dtype=np.float32).view(np.uint32))
        for w in ws:
            w.free()
        out.free()
        proj.workspace.free()


# ---- the same generators over row lengths that leave the usual kernels ----------------------------

AWKWARD_BATCHED = [2816, 4864, 5632, 6912, 11008, 13824, 18944, 25600]     # 11, 19, 22, 27, 43, 54, 74, 100 blocks of 256
LONG_SINGLE = [16640, 17408, 18944, 22016, 25600, 27648, 28672, 32768]     # past the 16 384 columns a workgroup spans


@pytest.mark.parametrize("chunk", range(3))
def test_random_calls_over_awkward_row_lengths(ctx, chunk, monkeypatch):
    """Batched calls over rows whose blocks have no cut into equal spans (served as two column windows,
    or by the in-loop kernel, or decoded once), and single-token calls over rows longer than a
    workgroup spans (the two-halves form of the tile kernel, or the catch-all kernel)."""
    import sys
    me = sys.modules[__name__]
    rng = np.random.default_rng(20261300 + chunk)
    monkeypatch.setattr(me, "ROW_LENGTHS", AWKWARD_BATCHED)
    for i in range(20):
        c = batched_case(rng)
        if c["batch"] * c["ldo"] > 30_000_000:
            continue
        say("random batched call, awkward row length", chunk, i, c)
        run_batched_case(ctx, c, seed=(chunk * 100 + i) * 16 + 13000)
    monkeypatch.setattr(me, "ROW_LENGTHS", LONG_SINGLE)
    for i in range(30):
        c = single_case(rng)
        say("random single-token call, long rows", chunk, i, c)
        run_single_case(ctx, c, seed=(chunk * 100 + i) * 16 + 14000)
