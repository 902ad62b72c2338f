"""Independent numpy statements of the block formats, written from the ggml format description
(block_q8_0 / block_q4_0 / block_q4_K and get_scale_min_k4), NOT from the oracle's C text: they
exist so the oracle is checked against something that was not typed from the same lines.
All arithmetic is float32, one rounding per operation, no fused multiply-add.
"""
from __future__ import annotations

import numpy as np

F32 = np.float32


def half_bits_to_f32(bits: np.ndarray) -> np.ndarray:
    return np.asarray(bits, dtype=np.uint16).view(np.float16).astype(np.float32)


def dequant_q8_0(raw: np.ndarray) -> np.ndarray:
    b = raw.reshape(-1, 34)
    d = half_bits_to_f32(b[:, 0:2].copy().view(np.uint16)[:, 0])
    q = b[:, 2:].view(np.int8).astype(np.float32)
    with np.errstate(invalid="ignore", over="ignore"):
        return (q * d[:, None]).astype(np.float32).reshape(-1)


def dequant_q4_0(raw: np.ndarray) -> np.ndarray:
    b = raw.reshape(-1, 18)
    d = half_bits_to_f32(b[:, 0:2].copy().view(np.uint16)[:, 0])
    qs = b[:, 2:]
    lo = (qs & 0x0F).astype(np.int32) - 8
    hi = (qs >> 4).astype(np.int32) - 8
    q = np.concatenate([lo, hi], axis=1).astype(np.float32)
    with np.errstate(invalid="ignore", over="ignore"):
        return (q * d[:, None]).astype(np.float32).reshape(-1)


def q4_k_scales_mins(scales12: np.ndarray):
    """get_scale_min_k4 for j = 0..7 over [..., 12] scale bytes -> two [..., 8] integer arrays."""
    s = scales12.astype(np.int32)
    sc = np.empty(s.shape[:-1] + (8,), dtype=np.int32)
    mn = np.empty_like(sc)
    for j in range(4):
        sc[..., j] = s[..., j] & 63
        mn[..., j] = s[..., j + 4] & 63
    for j in range(4, 8):
        sc[..., j] = (s[..., j + 4] & 0xF) | ((s[..., j - 4] >> 6) << 4)
        mn[..., j] = (s[..., j + 4] >> 4) | ((s[..., j] >> 6) << 4)
    return sc, mn


def dequant_q4_k(raw: np.ndarray) -> np.ndarray:
    b = raw.reshape(-1, 144)
    nb = b.shape[0]
    d = half_bits_to_f32(b[:, 0:2].copy().view(np.uint16)[:, 0])
    dmin = half_bits_to_f32(b[:, 2:4].copy().view(np.uint16)[:, 0])
    sc, mn = q4_k_scales_mins(b[:, 4:16])
    qs = b[:, 16:].reshape(nb, 4, 32)
    out = np.empty((nb, 8, 32), dtype=np.float32)
    with np.errstate(invalid="ignore", over="ignore"):
        for j in range(8):
            nib = (qs[:, j // 2, :] >> (4 * (j % 2))) & 0xF
            d1 = (d * sc[:, j].astype(np.float32)).astype(np.float32)
            m1 = (dmin * mn[:, j].astype(np.float32)).astype(np.float32)
            t = (d1[:, None] * nib.astype(np.float32)).astype(np.float32)
            out[:, j, :] = (t - m1[:, None]).astype(np.float32)
    return out.reshape(-1)


def dequant_q5_k(raw: np.ndarray) -> np.ndarray:
    """ggml's dequantize_row_q5_K, vectorised: sub-block j of 32 takes its low four bits from
    nibble j % 2 of qs[32 (j // 2) ...], its fifth bit from bit j of qh, scale and min as Q4_K;
    w = d * sc * q - dmin * m with every product and the difference rounded to fp32."""
    b = raw.reshape(-1, 176)
    nb = b.shape[0]
    d = half_bits_to_f32(b[:, 0:2].copy().view(np.uint16)[:, 0])
    dmin = half_bits_to_f32(b[:, 2:4].copy().view(np.uint16)[:, 0])
    sc, mn = q4_k_scales_mins(b[:, 4:16])
    qh = b[:, 16:48].astype(np.int32)
    qs = b[:, 48:].reshape(nb, 4, 32).astype(np.int32)
    out = np.empty((nb, 8, 32), dtype=np.float32)
    with np.errstate(invalid="ignore", over="ignore"):
        for j in range(8):
            q = ((qs[:, j // 2, :] >> (4 * (j % 2))) & 0xF) + (((qh >> j) & 1) << 4)
            d1 = (d * sc[:, j].astype(np.float32)).astype(np.float32)
            m1 = (dmin * mn[:, j].astype(np.float32)).astype(np.float32)
            t = (d1[:, None] * q.astype(np.float32)).astype(np.float32)
            out[:, j, :] = (t - m1[:, None]).astype(np.float32)
    return out.reshape(-1)


def dequant_q6_k(raw: np.ndarray) -> np.ndarray:
    """ggml's dequantize_row_q6_K, vectorised: per half of 128, y[l + 32 g] for l < 32 takes its low
    four bits from ql (plane g % 2, nibble g // 2), bits 4-5 from qh >> 2 g, the scale
    sc[l // 16 + 2 g]; w = d * sc * (q - 32) with every product rounded to fp32."""
    b = raw.reshape(-1, 210)
    nb = b.shape[0]
    ql = b[:, 0:128].reshape(nb, 2, 2, 32).astype(np.int32)       # [block, half, plane, l]
    qh = b[:, 128:192].reshape(nb, 2, 32).astype(np.int32)        # [block, half, l]
    sc = b[:, 192:208].copy().view(np.int8).reshape(nb, 2, 8).astype(np.float32)
    d = half_bits_to_f32(b[:, 208:210].copy().view(np.uint16)[:, 0])
    out = np.empty((nb, 2, 4, 32), dtype=np.float32)
    l16 = np.arange(32) // 16
    with np.errstate(invalid="ignore", over="ignore"):
        for g in range(4):
            low = (ql[:, :, g % 2, :] >> (4 * (g // 2))) & 0xF
            q = (low | (((qh >> (2 * g)) & 3) << 4)) - 32
            scale = sc[:, :, l16 + 2 * g]                          # [block, half, l]
            t = (d[:, None, None] * scale).astype(np.float32)
            out[:, :, g, :] = (t * q.astype(np.float32)).astype(np.float32)
    return out.reshape(-1)


def dequant_q4_1(raw: np.ndarray) -> np.ndarray:
    """ggml's dequantize_row_q4_1: y[j] = (qs[j] & 0xF) * d + m, y[j + 16] = (qs[j] >> 4) * d + m."""
    b = raw.reshape(-1, 20)
    d = half_bits_to_f32(b[:, 0:2].copy().view(np.uint16)[:, 0])
    m = half_bits_to_f32(b[:, 2:4].copy().view(np.uint16)[:, 0])
    q = np.concatenate([b[:, 4:] & 0x0F, b[:, 4:] >> 4], axis=1).astype(np.float32)
    with np.errstate(invalid="ignore", over="ignore"):
        return ((q * d[:, None]).astype(np.float32) + m[:, None]).astype(np.float32).reshape(-1)


def dequant_q5_0(raw: np.ndarray) -> np.ndarray:
    """ggml's dequantize_row_q5_0: qh is a little-endian 32-bit word; y[j] takes bit j of it as its
    fifth bit and the low nibble of qs[j], y[j + 16] bit j + 16 and the high nibble; w = (q - 16) d."""
    b = raw.reshape(-1, 22)
    d = half_bits_to_f32(b[:, 0:2].copy().view(np.uint16)[:, 0])
    qh = b[:, 2:6].copy().view("<u4")[:, 0].astype(np.int64)
    bits = (qh[:, None] >> np.arange(32)[None, :]) & 1
    nib = np.concatenate([b[:, 6:] & 0x0F, b[:, 6:] >> 4], axis=1).astype(np.int64)
    q = ((nib | (bits << 4)) - 16).astype(np.float32)
    with np.errstate(invalid="ignore", over="ignore"):
        return (d[:, None] * q).astype(np.float32).reshape(-1)


KVALUES_IQ4NL = np.array([-127, -104, -83, -65, -49, -35, -22, -10, 1, 13, 25, 38, 53, 69, 89, 113],
                         dtype=np.float32)


def dequant_iq4_xs(raw: np.ndarray) -> np.ndarray:
    """ggml's dequantize_row_iq4_xs: for group ib of 32, ls = low four bits from scales_l[ib / 2]
    (nibble ib % 2) | two bits of scales_h at 2 ib << 4, dl = d * (ls - 32); y[j] = dl *
    kvalues_iq4nl[qs[j] & 0xF], y[j + 16] = dl * kvalues_iq4nl[qs[j] >> 4] over the group's 16 bytes."""
    b = raw.reshape(-1, 136)
    nb = b.shape[0]
    d = half_bits_to_f32(b[:, 0:2].copy().view(np.uint16)[:, 0])
    scales_h = b[:, 2:4].copy().view("<u2")[:, 0].astype(np.int32)
    scales_l = b[:, 4:8].astype(np.int32)
    qs = b[:, 8:].reshape(nb, 8, 16)
    out = np.empty((nb, 8, 32), dtype=np.float32)
    with np.errstate(invalid="ignore", over="ignore"):
        for ib in range(8):
            ls = ((scales_l[:, ib // 2] >> (4 * (ib % 2))) & 0xF) | (((scales_h >> (2 * ib)) & 3) << 4)
            dl = (d * (ls - 32).astype(np.float32)).astype(np.float32)
            out[:, ib, 0:16] = (dl[:, None] * KVALUES_IQ4NL[qs[:, ib, :] & 0xF]).astype(np.float32)
            out[:, ib, 16:32] = (dl[:, None] * KVALUES_IQ4NL[qs[:, ib, :] >> 4]).astype(np.float32)
    return out.reshape(-1)


DEQUANT = {8: dequant_q8_0, 2: dequant_q4_0, 12: dequant_q4_k, 13: dequant_q5_k, 14: dequant_q6_k,
           3: dequant_q4_1, 6: dequant_q5_0, 23: dequant_iq4_xs}


def scalar_dot_rows(w_deq: np.ndarray, x: np.ndarray) -> np.ndarray:
    """Strictly sequential float32 dot of every row of ``w_deq`` [d x n] with ``x`` [n]."""
    d, n = w_deq.shape
    acc = np.zeros(d, dtype=np.float32)
    for j in range(n):
        acc = (acc + (w_deq[:, j] * x[j]).astype(np.float32)).astype(np.float32)
    return acc


def _fma32(a: np.ndarray, b: np.ndarray, c: np.ndarray) -> np.ndarray:
    """fma in float32 for operands whose exact a*b+c fits a double (|terms| small): the product of
    two float32 values is exact in float64, and one float64 add then one rounding to float32
    differs from a true fma only by double rounding, which the callers' tolerance absorbs."""
    return (a.astype(np.float64) * b.astype(np.float64) + c.astype(np.float64)).astype(np.float32)


def vector_lane_values(t: int, raw: np.ndarray, x: np.ndarray, bits: int) -> np.ndarray:
    """Lane accumulators of the reference's vector dot for one row, before reduceLanes."""
    m = None
    if t == 8:
        b = raw.reshape(-1, 34)
        wf = b[:, 2:].view(np.int8).astype(np.float32)
    elif t == 3:
        b = raw.reshape(-1, 20)
        wf = np.concatenate([b[:, 4:] & 0xF, b[:, 4:] >> 4], axis=1).astype(np.float32)
        m = half_bits_to_f32(b[:, 2:4].copy().view(np.uint16)[:, 0])
    else:
        b = raw.reshape(-1, 18)
        qs = b[:, 2:]
        wf = np.concatenate([(qs & 0xF).astype(np.int32) - 8, (qs >> 4).astype(np.int32) - 8],
                            axis=1).astype(np.float32)
    d = half_bits_to_f32(b[:, 0:2].copy().view(np.uint16)[:, 0])
    lanes = bits // 32
    val = np.zeros(lanes, dtype=np.float32)
    xb = x.reshape(-1, 32)
    for k in range(b.shape[0]):
        halves = [(0, 32)] if bits == 256 else [(0, 16), (16, 32)]
        for lo, hi in halves:
            p = (xb[k, lo:hi] * wf[k, lo:hi]).astype(np.float32).reshape(4, lanes)
            s = ((p[0] + p[1]).astype(np.float32) + p[2]).astype(np.float32)
            s = (s + p[3]).astype(np.float32)
            val = _fma32(s, np.full(lanes, d[k], dtype=np.float32), val)
            if m is not None:   # Q4_1: the activation slices, summed the same way, times the minimum
                a = xb[k, lo:hi].reshape(4, lanes)
                sa = ((a[0] + a[1]).astype(np.float32) + a[2]).astype(np.float32)
                sa = (sa + a[3]).astype(np.float32)
                val = _fma32(sa, np.full(lanes, m[k], dtype=np.float32), val)
    return val


def block_sum_dot_rows(w_deq: np.ndarray, x: np.ndarray, group: int = 32) -> np.ndarray:
    """Rows of ``w_deq`` [d x n] times ``x``: each run of ``group`` products summed sequentially in
    float32 from zero, the runs' sums added sequentially to the result."""
    d, n = w_deq.shape
    acc = np.zeros(d, dtype=np.float32)
    for g in range(n // group):
        part = np.zeros(d, dtype=np.float32)
        for j in range(g * group, (g + 1) * group):
            part = (part + (w_deq[:, j] * x[j]).astype(np.float32)).astype(np.float32)
        acc = (acc + part).astype(np.float32)
    return acc
