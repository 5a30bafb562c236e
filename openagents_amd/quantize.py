"""Host-side GGUF quantizers for the two closed-form formats (Q4_0, Q8_0), vectorized in numpy.

These are the producers of synthetic weights for benchmarks and examples: fp32 [n, k] ->
uint8 [n, k/32 * block_bytes] of GGUF blocks.  They restate the published block definitions
(Q8_0: d = amax/127, q = round-half-away(x/d); Q4_0: d = (signed max)/-8,
q = min(15, trunc(x/d + 8.5)), low nibbles = elements 0..15, high nibbles = 16..31) and are
checked bit-for-bit against the CPU oracle in tests/test_quantize_host.py.
"""
from __future__ import annotations

import numpy as np


def _blocks(x: np.ndarray) -> np.ndarray:
    x = np.ascontiguousarray(x, dtype=np.float32)
    if x.ndim != 2 or x.shape[1] % 32:
        raise ValueError("expected fp32 [n, k] with k a multiple of 32")
    return x.reshape(x.shape[0], x.shape[1] // 32, 32)


def quantize_q8_0(x: np.ndarray) -> np.ndarray:
    xb = _blocks(x)
    n, nb, _ = xb.shape
    amax = np.abs(xb).max(axis=2)
    d = (amax / np.float32(127.0)).astype(np.float32)
    with np.errstate(divide="ignore"):
        inv = np.where(d != 0, np.float32(1.0) / d, np.float32(0.0)).astype(np.float32)
    v = (xb * inv[:, :, None]).astype(np.float32)
    q = (np.sign(v) * np.floor(np.abs(v).astype(np.float64) + 0.5)).astype(np.int8)   # round half away from zero
    out = np.empty((n, nb, 34), dtype=np.uint8)
    out[:, :, 0:2] = d.astype(np.float16).view(np.uint8).reshape(n, nb, 2)
    out[:, :, 2:] = q.view(np.uint8)
    return out.reshape(n, nb * 34)


def quantize_q4_0(x: np.ndarray) -> np.ndarray:
    xb = _blocks(x)
    n, nb, _ = xb.shape
    idx = np.abs(xb).argmax(axis=2)                               # first element of largest magnitude
    vmax = np.take_along_axis(xb, idx[:, :, None], axis=2)[:, :, 0]
    d = (vmax / np.float32(-8.0)).astype(np.float32)
    with np.errstate(divide="ignore"):
        inv = np.where(d != 0, np.float32(1.0) / d, np.float32(0.0)).astype(np.float32)
    v = ((xb * inv[:, :, None]).astype(np.float32) + np.float32(8.5)).astype(np.float32)
    q = np.minimum(15, v.astype(np.int32).astype(np.int8).astype(np.int32)).astype(np.uint8)   # trunc, int8 wrap, clamp
    out = np.empty((n, nb, 18), dtype=np.uint8)
    out[:, :, 0:2] = d.astype(np.float16).view(np.uint8).reshape(n, nb, 2)
    out[:, :, 2:] = q[:, :, :16] | (q[:, :, 16:] << 4)
    return out.reshape(n, nb * 18)
