"""Seeded synthetic weights and activations of the benchmark's shapes.

Block value distributions:
  Q8_0  fp16 d ~ U(1e-3, 2e-2) per block, 32 int8 ~ U{-127..127}
  Q4_0  fp16 d ~ U(1e-3, 2e-2) per block, 16 bytes of nibbles ~ U{0..15}
  Q4_K  fp16 d ~ U(1e-3, 2e-2)/63, fp16 dmin ~ U(1e-3, 2e-2)*8/63 per super-block (so the largest
        weight magnitude d*63*15 stays near 0.3 and the minimum term roughly centres the range),
        8 (scale, min) pairs ~ U{0..63} packed into the 12 scale bytes, 128 bytes of nibbles
  Q4_1  fp16 d ~ U(1e-3, 2e-2), fp16 m = -7.5 d * U(0.5, 1.5) per block (the minimum roughly centres
        the range), 16 bytes of nibbles
  Q5_0  fp16 d ~ U(5e-4, 1e-2) per block, 4 bytes of fifth bits, 16 bytes of nibbles
  IQ4_XS fp16 d ~ U(2e-5, 1e-4) per super-block (largest weight d*31*127 near 0.4), 8 six-bit group
        scales split over scales_h / scales_l, 128 bytes of nibbles
  Q5_K  as Q4_K with d and dmin halved (values reach 31), plus 32 bytes of fifth bits
  Q6_K  fp16 d ~ U(2e-5, 1e-4) per super-block (largest weight d*127*32 near 0.4), 16 signed
        scales ~ U{-128..127}, 128 + 64 bytes of quant bits
  x     fp32 ~ N(0, 1)
One seed makes one tensor (numpy PCG64).
"""
from __future__ import annotations

import numpy as np

from .ggml import GGMLType


def _scales_f16(rng: np.random.Generator, count: int, lo: float, hi: float) -> np.ndarray:
    return rng.uniform(lo, hi, size=count).astype(np.float32).astype(np.float16).view(np.uint16)


def pack_q4_k_scales(sc: np.ndarray, m: np.ndarray) -> np.ndarray:
    """Inverse of Q4_KFloatTensor.getScaleK4/getMinK4: [..., 8] scales and mins -> [..., 12] bytes."""
    sc = sc.astype(np.uint8)
    m = m.astype(np.uint8)
    out = np.empty(sc.shape[:-1] + (12,), dtype=np.uint8)
    out[..., 0:4] = (sc[..., 0:4] & 63) | ((sc[..., 4:8] >> 4) << 6)
    out[..., 4:8] = (m[..., 0:4] & 63) | ((m[..., 4:8] >> 4) << 6)
    out[..., 8:12] = (sc[..., 4:8] & 0xF) | ((m[..., 4:8] & 0xF) << 4)
    return out


def weight(t: GGMLType, rows: int, cols: int, seed: int) -> np.ndarray:
    """Raw GGUF blocks of a ``[rows x cols]`` weight, row-major, as a flat uint8 array."""
    t = GGMLType(t)
    if cols % t.block_elems:
        raise ValueError(f"cols={cols} is not a multiple of the {t.name} block ({t.block_elems})")
    rng = np.random.default_rng(seed)
    blocks = rows * (cols // t.block_elems)
    raw = np.empty((blocks, t.block_bytes), dtype=np.uint8)
    if t == GGMLType.Q8_0:
        raw[:, 0:2] = _scales_f16(rng, blocks, 1e-3, 2e-2).view(np.uint8).reshape(blocks, 2)
        raw[:, 2:] = rng.integers(-127, 128, size=(blocks, 32), dtype=np.int8).view(np.uint8)
    elif t == GGMLType.Q4_0:
        raw[:, 0:2] = _scales_f16(rng, blocks, 1e-3, 2e-2).view(np.uint8).reshape(blocks, 2)
        raw[:, 2:] = rng.integers(0, 256, size=(blocks, 16), dtype=np.uint8)
    elif t == GGMLType.Q4_1:
        d = rng.uniform(1e-3, 2e-2, size=blocks).astype(np.float32)
        m = (-7.5 * d * rng.uniform(0.5, 1.5, size=blocks)).astype(np.float32)
        raw[:, 0:2] = d.astype(np.float16).view(np.uint16).view(np.uint8).reshape(blocks, 2)
        raw[:, 2:4] = m.astype(np.float16).view(np.uint16).view(np.uint8).reshape(blocks, 2)
        raw[:, 4:] = rng.integers(0, 256, size=(blocks, 16), dtype=np.uint8)
    elif t == GGMLType.Q5_0:
        raw[:, 0:2] = _scales_f16(rng, blocks, 5e-4, 1e-2).view(np.uint8).reshape(blocks, 2)
        raw[:, 2:] = rng.integers(0, 256, size=(blocks, 20), dtype=np.uint8)
    elif t == GGMLType.IQ4_XS:
        raw[:, 0:2] = _scales_f16(rng, blocks, 2e-5, 1e-4).view(np.uint8).reshape(blocks, 2)
        raw[:, 2:] = rng.integers(0, 256, size=(blocks, 134), dtype=np.uint8)
    elif t == GGMLType.Q5_K:
        raw[:, 0:2] = _scales_f16(rng, blocks, 5e-4 / 63, 1e-2 / 63).view(np.uint8).reshape(blocks, 2)
        raw[:, 2:4] = _scales_f16(rng, blocks, 8e-3 / 63, 16e-2 / 63).view(np.uint8).reshape(blocks, 2)
        sc = rng.integers(0, 64, size=(blocks, 8), dtype=np.uint8)
        m = rng.integers(0, 64, size=(blocks, 8), dtype=np.uint8)
        raw[:, 4:16] = pack_q4_k_scales(sc, m)
        raw[:, 16:] = rng.integers(0, 256, size=(blocks, 160), dtype=np.uint8)
    elif t == GGMLType.Q6_K:
        raw[:, 0:192] = rng.integers(0, 256, size=(blocks, 192), dtype=np.uint8)
        raw[:, 192:208] = rng.integers(-128, 128, size=(blocks, 16), dtype=np.int8).view(np.uint8)
        raw[:, 208:210] = _scales_f16(rng, blocks, 2e-5, 1e-4).view(np.uint8).reshape(blocks, 2)
    else:
        raw[:, 0:2] = _scales_f16(rng, blocks, 1e-3 / 63, 2e-2 / 63).view(np.uint8).reshape(blocks, 2)
        raw[:, 2:4] = _scales_f16(rng, blocks, 8e-3 / 63, 16e-2 / 63).view(np.uint8).reshape(blocks, 2)
        sc = rng.integers(0, 64, size=(blocks, 8), dtype=np.uint8)
        m = rng.integers(0, 64, size=(blocks, 8), dtype=np.uint8)
        raw[:, 4:16] = pack_q4_k_scales(sc, m)
        raw[:, 16:] = rng.integers(0, 256, size=(blocks, 128), dtype=np.uint8)
    return raw.reshape(-1)


def activations(shape, seed: int) -> np.ndarray:
    return np.random.default_rng(seed).standard_normal(size=shape, dtype=np.float32)
