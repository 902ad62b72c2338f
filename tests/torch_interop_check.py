"""PyTorch as plumbing, run as a program of its own (tests/test_gpu_torch_interop.py starts it):
activations and results are torch tensors whose data_ptr goes to the C ABI, the context borrows a
torch stream, and the kernels torch enqueues on that stream before and after the call are ordered
with it -- no synchronization between the three."""
import ctypes as C
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "tests"))


def main() -> int:
    import torch

    from gpu_util import magnitude, rel_err
    from jitllm_amd import _lib as L, synthetic
    from jitllm_amd.runtime import Context
    from oracle import pyoracle as O
    untouched = np.float32(-12345.5)
    t, d, n, rows = O.Q4_K, 3072, 2048, 24
    raw = synthetic.weight(t, d, n, seed=9880)
    X = synthetic.activations((rows, n), seed=9881)
    s = torch.cuda.Stream()
    c = Context(0, stream=s.cuda_stream)
    w = c.load_weight(t, raw, d, n)
    lib = c._lib
    nbytes = lib.jl_gemm_workspace_bytes(rows, n, d, L.JL_MATH_DEFAULT)
    with torch.cuda.stream(s):
        half = torch.from_numpy(X / 2).to("cuda")
        x = half * 2                                   # torch's kernel, on s, produces the input
        out = torch.full((rows, d), float(untouched), device="cuda")
        ws = torch.empty(max(nbytes, 256), dtype=torch.uint8, device="cuda")
        weights = (C.c_void_p * 1)(w.handle)
        L.check(lib.jl_gemm(c.handle, weights, 1, C.c_void_p(x.data_ptr()), C.c_void_p(out.data_ptr()), rows, rows, d, 0,
                            L.JL_STORE, L.JL_MATH_DEFAULT, C.c_void_p(ws.data_ptr()), nbytes))
        doubled = out * 2                              # and torch's next kernel consumes the result
        got = doubled.cpu().numpy() / 2
    edge = 128
    part = raw[:edge * (raw.size // d)]
    ref = O.matmul_batch(t, part, X, edge, n)
    err = rel_err(got[:, :edge], ref, magnitude(t, part, X, edge, n))
    ok = err < 2e-3 and bool(np.all(got != untouched))
    print("torch interop: rel err %.3g, %s" % (err, "ok" if ok else "FAILED"), flush=True)
    w.free()
    c.close()
    return 0 if ok else 1


if __name__ == "__main__":
    sys.exit(main())
