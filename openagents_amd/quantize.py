"""Host-side GGUF weight quantizers: fp32 [n, k] -> uint8 [n, row_bytes] of GGUF blocks.

Thin wrappers over the library's native quantizer (`psn_quantize_rows`, host code, no device
needed), which restates the published reference quantizers -- closed forms for Q4_0 / Q8_0, the
weighted least-squares scale searches for Q4_K / Q5_K / Q6_K -- so the bytes are the ones the
reference's CPU path produces from the same fp32 rows.  These are the producers of the seeded
synthetic weights of the benchmarks and examples, and the import step for fp32 checkpoints.
"""
from __future__ import annotations

import ctypes as C
import os

import numpy as np

from . import _ffi
from ._ffi import Q4_0, Q4_K, Q5_K, Q6_K, Q8_0


def default_threads() -> int:
    try:
        return max(1, len(os.sched_getaffinity(0)))
    except AttributeError:
        return max(1, os.cpu_count() or 1)


def quantize(qtype: int, x: np.ndarray, threads: int | None = None) -> np.ndarray:
    """fp32 [n, k] -> uint8 [n, psn_row_bytes(qtype, k)].  Raises ValueError on a ragged shape."""
    lib = _ffi.load()
    x = np.ascontiguousarray(x, dtype=np.float32)
    if x.ndim != 2 or x.shape[0] == 0:
        raise ValueError("expected a non-empty fp32 [n, k] array")
    n, k = x.shape
    rb = lib.psn_row_bytes(qtype, k)
    if rb < 0:
        raise ValueError(lib.psn_last_error().decode(errors="replace"))
    out = np.empty((n, rb), dtype=np.uint8)
    rc = lib.psn_quantize_rows(qtype, C.c_void_p(x.ctypes.data), n, k, C.c_void_p(out.ctypes.data), out.nbytes,
                               threads if threads is not None else default_threads())
    if rc < 0:
        raise ValueError(lib.psn_last_error().decode(errors="replace"))
    return out


def quantize_q4_0(x: np.ndarray, threads: int | None = None) -> np.ndarray:
    return quantize(Q4_0, x, threads)


def quantize_q8_0(x: np.ndarray, threads: int | None = None) -> np.ndarray:
    return quantize(Q8_0, x, threads)


def quantize_q4_K(x: np.ndarray, threads: int | None = None) -> np.ndarray:
    return quantize(Q4_K, x, threads)


def quantize_q5_K(x: np.ndarray, threads: int | None = None) -> np.ndarray:
    return quantize(Q5_K, x, threads)


def quantize_q6_K(x: np.ndarray, threads: int | None = None) -> np.ndarray:
    return quantize(Q6_K, x, threads)


def dequantize(qtype: int, blocks: np.ndarray, k: int) -> np.ndarray:
    """uint8 [n, psn_row_bytes(qtype, k)] (or one flat row) -> fp32 [n, k], the reference's dequantize_row_* values."""
    lib = _ffi.load()
    rb = lib.psn_row_bytes(qtype, k)
    if rb < 0:
        raise ValueError(lib.psn_last_error().decode(errors="replace"))
    b = np.ascontiguousarray(blocks, dtype=np.uint8).reshape(-1)
    if b.size == 0 or b.size % rb:
        raise ValueError(f"{b.size} bytes is not a whole number of {rb}-byte rows")
    n = b.size // rb
    out = np.empty((n, k), dtype=np.float32)
    rc = lib.psn_dequantize_rows(qtype, C.c_void_p(b.ctypes.data), n, k, C.c_void_p(out.ctypes.data), out.size)
    if rc < 0:
        raise ValueError(lib.psn_last_error().decode(errors="replace"))
    return out
