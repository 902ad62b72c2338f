"""Helpers shared by the GPU parity tests: error metrics and oracle references."""
from __future__ import annotations

import sys

import numpy as np

import np_models as NP
from oracle import pyoracle as O


def say(*parts) -> None:
    """Names the case before its GPU step, flushed, so a fault leaves the culprit on stdout."""
    print("[gpu-case]", *parts, flush=True)


def magnitude(t: int, raw: np.ndarray, X: np.ndarray, d: int, n: int) -> np.ndarray:
    """sum_j |w_ij x_bj| in float64, [B x d] (or [d] for a vector)."""
    w = np.abs(NP.DEQUANT[t](raw).reshape(d, n).astype(np.float64))
    X = np.asarray(X, dtype=np.float64)
    if X.ndim == 1:
        return w @ np.abs(X)
    return np.abs(X) @ w.T


def rel_err(got: np.ndarray, ref: np.ndarray, mag: np.ndarray) -> float:
    """max_i |got_i - ref_i| / sum_j |w_ij x_j|: the bound the path is held to (1e-3; 2e-3 on the
    fp16-MFMA path).  A plain |d|/|ref| blows up on outputs that cancel to nearly zero."""
    return float(np.max(np.abs(got.astype(np.float64) - ref.astype(np.float64)) / np.maximum(mag, 1e-30)))


def reference_tolerance_ok(got: np.ndarray, want: np.ndarray) -> np.ndarray:
    """The reference's own kernel-test form: |got - want| <= max(1e-3, 1e-4 |want|)
    (NativeQuantizedKernelAccelTest.java:170)."""
    tol = np.maximum(np.float32(1e-3), np.abs(want) * np.float32(1e-4))
    return np.abs(got - want) <= tol


def bits_equal(a: np.ndarray, b: np.ndarray) -> bool:
    a = np.asarray(a, np.float32).reshape(-1)
    b = np.asarray(b, np.float32).reshape(-1)
    nan = np.isnan(a)
    if not np.array_equal(nan, np.isnan(b)):
        return False
    return np.array_equal(a.view(np.uint32)[~nan], b.view(np.uint32)[~nan])
