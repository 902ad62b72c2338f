"""Input recipes of the reference's own tests, regenerated from their seeds.

Each function cites the reference test it restates (T = src/test/java/org/beehive/jitllm).  The
bytes come from a bit-faithful java.util.Random (oracle/jitllm_oracle.c), so they are the bytes
the reference's JUnit runs see.
"""
from __future__ import annotations

import numpy as np

from oracle import pyoracle as O

N_PROBE, D_PROBE = 512, 37  # T/backend/tornado/kernels/NativeQuantizedKernelAccelTest.java:56-58

SPECIAL_HALVES = [0x0000, 0x8000, 0x0001, 0x03FF, 0x3C00, 0xBC00, 0x7BFF, 0xFBFF]
PAYLOAD_PATTERNS = [0x00, 0xFF, 0xAA, 0x55]

SCALE_OFFSETS = {O.Q4_0: [0], O.Q8_0: [0], O.Q4_K: [0, 2], O.Q5_K: [0, 2], O.Q6_K: [208],
                 O.Q4_1: [0, 2], O.Q5_0: [0], O.IQ4_XS: [0]}
TYPE_NAMES = {O.Q4_0: "Q4_0", O.Q8_0: "Q8_0", O.Q4_K: "Q4_K", O.Q5_K: "Q5_K", O.Q6_K: "Q6_K",
              O.Q4_1: "Q4_1", O.Q5_0: "Q5_0", O.IQ4_XS: "IQ4_XS"}


def random_bytes(seed: int, n: int) -> np.ndarray:
    """``new Random(seed).nextBytes(raw)`` (Q4_0DecodeTest.java:41-44, Q4_KDecodeTest.java:35-39)."""
    return O.JavaRandom(seed).next_bytes(n)


def adversarial_blocks(t: int, blocks: int, seed: int) -> np.ndarray:
    """T/backend/tornado/kernels/QuantizedDeviceDecodeParityTest.java:98-121."""
    bb = O.block_bytes(t)
    raw = random_bytes(seed, blocks * bb)
    for b in range(blocks):
        base = b * bb
        if b % 4 != 3:
            raw[base:base + bb] = PAYLOAD_PATTERNS[b % 4]
        for h, off in enumerate(SCALE_OFFSETS[t]):
            half = SPECIAL_HALVES[(b + h) % 8]
            raw[base + off] = half & 0xFF
            raw[base + off + 1] = (half >> 8) & 0xFF
    return raw


def probe_blocks(t: int, seed: int, both_scales: bool = False, n: int = N_PROBE,
                 d: int = D_PROBE) -> np.ndarray:
    """randomBlocks of NativeQuantizedKernelAccelTest.java:69-86 (scale bytes ``b & 0xFF, 0x2C``).

    ``both_scales`` is BatchProjectionTilingAccelTest.java:73-88, which writes offsets 0 and 2 for
    every type it covers.
    """
    bb = O.block_bytes(t)
    blocks = d * (n // O.block_elems(t))
    raw = random_bytes(seed, blocks * bb)
    offsets = [0, 2] if both_scales else SCALE_OFFSETS[t]
    for b in range(blocks):
        for off in offsets:
            raw[b * bb + off] = b & 0xFF
            raw[b * bb + off + 1] = 0x2C
    return raw


def probe_seed(name: str, base: int = 20260908) -> int:
    """``20260908L + name.hashCode()`` (NativeQuantizedKernelAccelTest.java:115)."""
    return base + O.java_string_hash(name)


def probe_x(n: int = N_PROBE) -> np.ndarray:
    """``x[i] = ((i % 7) - 3) * 0.25f`` (NativeQuantizedKernelAccelTest.java:117-120)."""
    i = np.arange(n)
    return (((i % 7) - 3) * np.float32(0.25)).astype(np.float32)


def batch_activation(width: int, n: int = N_PROBE) -> np.ndarray:
    """``activation(row, i)`` of BatchProjectionTilingAccelTest.java:99-101."""
    i = np.arange(n)[None, :]
    r = np.arange(width)[:, None]
    return ((((i + 3 * r) % 7) - 3) * np.float32(0.25)).astype(np.float32)


def int8_gemm_weights(n: int, k: int, seed: int) -> np.ndarray:
    """randomWeights of Qwen35Q8_0Int8ProjectionAccelTest.java:30-41."""
    rng = O.JavaRandom(seed)
    raw = rng.next_bytes(n * (k // 32) * 34)
    for b in range(n * (k // 32)):
        bits = 0x2000 | rng.next_int(0x400) | (0x8000 if rng.next_boolean() else 0)
        raw[b * 34] = bits & 0xFF
        raw[b * 34 + 1] = bits >> 8
    return raw


def int8_gemm_activations(m: int, k: int, seed: int) -> np.ndarray:
    """activations of Qwen35Q8_0Int8ProjectionAccelTest.java:51-58."""
    rng = O.JavaRandom(seed)
    return np.array([np.float32(rng.next_gaussian()) for _ in range(m * k)],
                    dtype=np.float32).reshape(m, k)
