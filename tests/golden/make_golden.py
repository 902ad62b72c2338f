"""Writes tests/golden/projection_golden.npz: inputs and expected outputs of the projection path.

Inputs are the reference's own test recipes (tests/fixtures.py restates them from their seeds) plus
a few seeded synthetic weights; expected outputs are what the CPU restatement of the reference's
host path (oracle/) returns for them.  The file travels to the GPU box, where the oracle's
outputs are compared with the HIP library's without recomputing anything, and it freezes the
oracle's behaviour: a later change to oracle/ that moves any of these values fails
tests/test_golden.py on the CPU.

Reference-held known answers that need no oracle (Q4_0DecodeTest.java:95-126) are kept as literals
in reference_known_answers.json next to this script.

Run from the repository root:  python tests/golden/make_golden.py
"""
from __future__ import annotations

import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "tests"))

import fixtures as FX  # noqa: E402
from jitllm_amd import synthetic  # noqa: E402
from oracle import pyoracle as O  # noqa: E402

OUT = os.path.join(os.path.dirname(os.path.abspath(__file__)), "projection_golden.npz")
TYPES = {"q8_0": O.Q8_0, "q4_0": O.Q4_0, "q4_k": O.Q4_K}


def main() -> None:
    data = {}
    x = FX.probe_x()
    data["probe_x"] = x
    for name, t in TYPES.items():
        # NativeQuantizedKernelAccelTest.java:69-135: probe blocks, N = 512, D = 37
        raw = FX.probe_blocks(t, FX.probe_seed(FX.TYPE_NAMES[t]))
        data[f"{name}.probe.raw"] = raw
        data[f"{name}.probe.dequant"] = O.dequant(t, raw[: 4 * O.block_bytes(t) * (256 // O.block_elems(t))])
        data[f"{name}.probe.matvec_scalar"] = O.matmul(t, raw, x, FX.D_PROBE, FX.N_PROBE, O.DOT_SCALAR)
        data[f"{name}.probe.matvec_vec256"] = O.matmul(t, raw, x, FX.D_PROBE, FX.N_PROBE, O.DOT_VEC256)
        # QuantizedDeviceDecodeParityTest.java:98-121: adversarial scale and payload patterns
        adv = FX.adversarial_blocks(t, 64, 20260907)
        data[f"{name}.adversarial.raw"] = adv
        data[f"{name}.adversarial.dequant"] = O.dequant(t, adv)
        # BatchProjectionTilingAccelTest.java:151-215: width 9, all rows active
        braw = FX.probe_blocks(t, 20260909 + O.java_string_hash(name.replace("_", "")), both_scales=(t == O.Q4_K))
        X = FX.batch_activation(9)
        data[f"{name}.batch.raw"] = braw
        data[f"{name}.batch.X"] = X
        data[f"{name}.batch.out"] = O.matmul_batch(t, braw, X, FX.D_PROBE, FX.N_PROBE)
        # a gate/up pair and a wider row, seeded synthetic blocks
        d, n = 40, 512
        w1 = synthetic.weight(t, d, n, seed=901)
        w3 = synthetic.weight(t, d, n, seed=902)
        xs = synthetic.activations(n, seed=903)
        g = O.matmul(t, w1, xs, d, n, O.DOT_SCALAR)
        u = O.matmul(t, w3, xs, d, n, O.DOT_SCALAR)
        data[f"{name}.gate_up.w1"] = w1
        data[f"{name}.gate_up.w3"] = w3
        data[f"{name}.gate_up.x"] = xs
        data[f"{name}.gate_up.out"] = O.swiglu(g, u)
    np.savez_compressed(OUT, **data)
    print(OUT, os.path.getsize(OUT), "bytes,", len(data), "arrays")


if __name__ == "__main__":
    main()
