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


def _f16_bytes(a: np.ndarray) -> np.ndarray:
    return np.ascontiguousarray(a.astype(np.float16)).view(np.uint8).reshape(a.shape + (2,))


def quantize_q4_K(x: np.ndarray) -> np.ndarray:
    """Q4_K producer without the reference encoder's iterative scale search: every 32-element
    sub-block gets the affine grid spanning [min(x, 0), max(x)], the eight scales and mins are
    re-quantized to 6 bits against the super-block maxima (fp16 d, dmin) and the nibbles are
    rounded against the re-quantized grid.  Any encoder that fills the fields in range is a legal
    GGUF producer; this one is for synthetic weights."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    if x.ndim != 2 or x.shape[1] % 256:
        raise ValueError("expected fp32 [n, k] with k a multiple of 256")
    n, k = x.shape
    nb = k // 256
    xb = x.reshape(n, nb, 8, 32)
    lo = np.minimum(xb.min(axis=3), 0.0)
    hi = xb.max(axis=3)
    scale = ((hi - lo) / np.float32(15.0)).astype(np.float32)
    mins = (-lo).astype(np.float32)
    max_scale = scale.max(axis=2)
    max_min = mins.max(axis=2)
    with np.errstate(divide="ignore", invalid="ignore"):
        inv_s = np.where(max_scale > 0, np.float32(63.0) / max_scale, 0).astype(np.float32)
        inv_m = np.where(max_min > 0, np.float32(63.0) / max_min, 0).astype(np.float32)
    ls = np.minimum(63, np.rint(inv_s[:, :, None] * scale)).astype(np.uint8)
    lm = np.minimum(63, np.rint(inv_m[:, :, None] * mins)).astype(np.uint8)
    d16 = (max_scale / np.float32(63.0)).astype(np.float16)
    m16 = (max_min / np.float32(63.0)).astype(np.float16)
    dl = d16.astype(np.float32)[:, :, None] * ls.astype(np.float32)
    ml = m16.astype(np.float32)[:, :, None] * lm.astype(np.float32)
    with np.errstate(divide="ignore", invalid="ignore"):
        q = np.where(dl[..., None] > 0, np.rint((xb + ml[..., None]) / dl[..., None]), 0)
    q = np.clip(q, 0, 15).astype(np.uint8).reshape(n, nb, 4, 2, 32)       # [chunk of 64][low/high half][32]
    out = np.zeros((n, nb, 144), dtype=np.uint8)
    out[:, :, 0:2] = _f16_bytes(d16.astype(np.float32))
    out[:, :, 2:4] = _f16_bytes(m16.astype(np.float32))
    out[:, :, 4:8] = (ls[:, :, 0:4] & 63) | ((ls[:, :, 4:8] >> 4) << 6)
    out[:, :, 8:12] = (lm[:, :, 0:4] & 63) | ((lm[:, :, 4:8] >> 4) << 6)
    out[:, :, 12:16] = (ls[:, :, 4:8] & 15) | ((lm[:, :, 4:8] & 15) << 4)
    out[:, :, 16:] = (q[:, :, :, 0, :] | (q[:, :, :, 1, :] << 4)).reshape(n, nb, 128)
    return out.reshape(n, nb * 144)


def quantize_q6_K(x: np.ndarray) -> np.ndarray:
    """Q6_K producer without the reference encoder's scale search: every 16-element group maps its
    extreme element to -32, the sixteen group scales are re-quantized to int8 against the
    super-block's fp16 d, and the 6-bit values are rounded against the re-quantized grid."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    if x.ndim != 2 or x.shape[1] % 256:
        raise ValueError("expected fp32 [n, k] with k a multiple of 256")
    n, k = x.shape
    nb = k // 256
    xb = x.reshape(n, nb, 16, 16)
    idx = np.abs(xb).argmax(axis=3)
    vmax = np.take_along_axis(xb, idx[..., None], axis=3)[..., 0]
    scale = (vmax / np.float32(-32.0)).astype(np.float32)                  # group scale, signed
    sidx = np.abs(scale).argmax(axis=2)
    smax = np.take_along_axis(scale, sidx[..., None], axis=2)[..., 0]
    with np.errstate(divide="ignore", invalid="ignore"):
        iscale = np.where(smax != 0, np.float32(-128.0) / smax, 0).astype(np.float32)
        d = np.where(iscale != 0, np.float32(1.0) / iscale, 0).astype(np.float32)
    d16 = d.astype(np.float16)
    sc = np.clip(np.rint(iscale[:, :, None] * scale), -128, 127).astype(np.int8)
    dl = d16.astype(np.float32)[:, :, None] * sc.astype(np.float32)
    with np.errstate(divide="ignore", invalid="ignore"):
        q = np.where(dl[..., None] != 0, np.rint(xb / dl[..., None]), 0)
    L = (np.clip(q, -32, 31) + 32).astype(np.uint8).reshape(n, nb, 2, 4, 32)   # [half][quarter][l]
    out = np.zeros((n, nb, 210), dtype=np.uint8)
    ql = out[:, :, 0:128].reshape(n, nb, 2, 64)
    qh = out[:, :, 128:192].reshape(n, nb, 2, 32)
    ql[:, :, :, 0:32] = (L[:, :, :, 0] & 15) | ((L[:, :, :, 2] & 15) << 4)
    ql[:, :, :, 32:64] = (L[:, :, :, 1] & 15) | ((L[:, :, :, 3] & 15) << 4)
    qh[:] = (L[:, :, :, 0] >> 4) | ((L[:, :, :, 1] >> 4) << 2) | ((L[:, :, :, 2] >> 4) << 4) | ((L[:, :, :, 3] >> 4) << 6)
    out[:, :, 192:208] = sc.view(np.uint8)
    out[:, :, 208:210] = _f16_bytes(d16.astype(np.float32))
    return out.reshape(n, nb * 210)
