"""ctypes binding of the CPU oracle (libpsn_oracle.so).

TEST INFRASTRUCTURE ONLY: imported by tests/, by __graft_entry__.smoke() and by the
cpu_baseline leg of bench.py.  The shipped package never imports this module.
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libpsn_oracle.so")

Q4_0, Q8_0, Q4_K, Q5_K, Q6_K, Q8_K = 2, 8, 12, 13, 14, 15
ACT_F32, ACT_Q8 = 0, 1
WEIGHT_TYPES = (Q4_0, Q8_0, Q4_K, Q5_K, Q6_K)
TYPE_NAMES = {Q4_0: "Q4_0", Q8_0: "Q8_0", Q4_K: "Q4_K", Q5_K: "Q5_K", Q6_K: "Q6_K", Q8_K: "Q8_K"}


def build(force: bool = False) -> str:
    """Compile the oracle with the Makefile beside it; returns the library path."""
    if force or not os.path.exists(_LIB_PATH):
        subprocess.check_call(["make", "-C", _HERE, "-B" if force else "-s", "libpsn_oracle.so"])
    return _LIB_PATH


_lib = None


def lib() -> C.CDLL:
    global _lib
    if _lib is None:
        build()
        L = C.CDLL(_LIB_PATH)
        vp, i32, i64, f32 = C.c_void_p, C.c_int32, C.c_int64, C.c_float
        L.orc_fp32_to_fp16.argtypes = [f32]; L.orc_fp32_to_fp16.restype = C.c_uint16
        L.orc_fp16_to_fp32.argtypes = [C.c_uint16]; L.orc_fp16_to_fp32.restype = f32
        L.orc_nearest_int.argtypes = [f32]; L.orc_nearest_int.restype = i32
        for name in ("orc_block_elems", "orc_block_bytes"):
            getattr(L, name).argtypes = [i32]; getattr(L, name).restype = i64
        L.orc_row_bytes.argtypes = [i32, i64]; L.orc_row_bytes.restype = i64
        L.orc_quantize_row.argtypes = [i32, vp, vp, i64]; L.orc_quantize_row.restype = i32
        L.orc_dequantize_row.argtypes = [i32, vp, vp, i64]; L.orc_dequantize_row.restype = i32
        L.orc_quantize_rows.argtypes = [i32, vp, vp, i64, i64, i32]; L.orc_quantize_rows.restype = i32
        L.orc_q4k_scale_min.argtypes = [vp, vp, vp]; L.orc_q4k_scale_min.restype = None
        L.orc_q4k_fit_subblock.argtypes = [vp, vp, C.POINTER(C.c_float)]; L.orc_q4k_fit_subblock.restype = f32
        L.orc_q6k_fit_subblock.argtypes = [vp, vp]; L.orc_q6k_fit_subblock.restype = f32
        L.orc_q5k_fit_subblock.argtypes = [vp, vp, C.POINTER(C.c_float)]; L.orc_q5k_fit_subblock.restype = f32
        L.orc_vec_dot_q.argtypes = [i32, vp, vp, i64]; L.orc_vec_dot_q.restype = f32
        L.orc_matvec.argtypes = [i32, i32, vp, vp, vp, i64, i64, i32, i32]; L.orc_matvec.restype = i32
        L.orc_matvec_f64.argtypes = [i32, vp, vp, vp, i64, i64, i32, i32]; L.orc_matvec_f64.restype = i32
        L.orc_prefill.argtypes = [i32, vp, vp, vp, i64, i64, i64, i32]; L.orc_prefill.restype = i32
        L.orc_max_threads.argtypes = []; L.orc_max_threads.restype = i32
        _lib = L
    return _lib


def _p(a: np.ndarray) -> C.c_void_p:
    return C.c_void_p(a.ctypes.data)


def max_threads() -> int:
    return int(lib().orc_max_threads())


def block_elems(qtype: int) -> int:
    return int(lib().orc_block_elems(qtype))


def block_bytes(qtype: int) -> int:
    return int(lib().orc_block_bytes(qtype))


def row_bytes(qtype: int, k: int) -> int:
    rb = int(lib().orc_row_bytes(qtype, k))
    if rb < 0:
        raise ValueError(f"k={k} is not a whole number of {TYPE_NAMES.get(qtype, qtype)} blocks")
    return rb


def fp32_to_fp16_bits(x: float) -> int:
    return int(lib().orc_fp32_to_fp16(C.c_float(x)))


def fp16_bits_to_fp32(h: int) -> float:
    return float(lib().orc_fp16_to_fp32(C.c_uint16(h)))


def nearest_int(x: float) -> int:
    return int(lib().orc_nearest_int(C.c_float(x)))


def quantize(qtype: int, x: np.ndarray, nthreads: int = 0) -> np.ndarray:
    """fp32 [n, k] (or [k]) -> uint8 [n, row_bytes] of GGUF blocks."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    x2 = x.reshape(1, -1) if x.ndim == 1 else x
    n, k = x2.shape
    rb = row_bytes(qtype, k)
    out = np.empty((n, rb), dtype=np.uint8)
    rc = lib().orc_quantize_rows(qtype, _p(x2), _p(out), n, k, nthreads or max_threads())
    if rc != 0:
        raise ValueError("orc_quantize_rows failed")
    return out[0] if x.ndim == 1 else out


def dequantize(qtype: int, blocks: np.ndarray, k: int) -> np.ndarray:
    """uint8 [n, row_bytes] (or [row_bytes]) -> fp32 [n, k]."""
    blocks = np.ascontiguousarray(blocks, dtype=np.uint8)
    b2 = blocks.reshape(1, -1) if blocks.ndim == 1 else blocks
    rb = row_bytes(qtype, k)
    assert b2.shape[1] == rb, (b2.shape, rb)
    out = np.empty((b2.shape[0], k), dtype=np.float32)
    for r in range(b2.shape[0]):
        rc = lib().orc_dequantize_row(qtype, C.c_void_p(b2[r].ctypes.data), C.c_void_p(out[r].ctypes.data), k)
        if rc != 0:
            raise ValueError("orc_dequantize_row failed")
    return out[0] if blocks.ndim == 1 else out


def q4k_scale_min(scales12: np.ndarray):
    s = np.ascontiguousarray(scales12, dtype=np.uint8)
    assert s.size == 12
    sc = np.zeros(8, dtype=np.uint8)
    mn = np.zeros(8, dtype=np.uint8)
    lib().orc_q4k_scale_min(_p(s), _p(sc), _p(mn))
    return sc, mn


def q4k_fit_subblock(x32: np.ndarray):
    """(scale, min, L[32]) of one Q4_K sub-block: x ~ scale * L - min."""
    x = np.ascontiguousarray(x32, dtype=np.float32)
    assert x.size == 32
    L = np.zeros(32, dtype=np.uint8)
    mn = C.c_float()
    sc = lib().orc_q4k_fit_subblock(_p(x), _p(L), C.byref(mn))
    return float(sc), float(mn.value), L


def q5k_fit_subblock(x32: np.ndarray):
    """(scale, min, L[32]) of one Q5_K sub-block: x ~ scale * L - min, L in 0..31."""
    x = np.ascontiguousarray(x32, dtype=np.float32)
    assert x.size == 32
    L = np.zeros(32, dtype=np.uint8)
    mn = C.c_float()
    sc = lib().orc_q5k_fit_subblock(_p(x), _p(L), C.byref(mn))
    return float(sc), float(mn.value), L


def q6k_fit_subblock(x16: np.ndarray):
    """(scale, L[16]) of one Q6_K sub-block: x ~ scale * (L - 32)."""
    x = np.ascontiguousarray(x16, dtype=np.float32)
    assert x.size == 16
    L = np.zeros(16, dtype=np.int8)
    sc = lib().orc_q6k_fit_subblock(_p(x), _p(L))
    return float(sc), L


def vec_dot_q(wtype: int, w_row: np.ndarray, xq_row: np.ndarray, k: int) -> float:
    w_row = np.ascontiguousarray(w_row, dtype=np.uint8)
    xq_row = np.ascontiguousarray(xq_row, dtype=np.uint8)
    return float(lib().orc_vec_dot_q(wtype, _p(w_row), _p(xq_row), k))


def matvec(wtype: int, scheme: int, W: np.ndarray, x: np.ndarray, n: int, k: int, nthreads: int = 0) -> np.ndarray:
    """W uint8 [n, row_bytes]; x fp32 [batch, k] or [k]; returns fp32 [batch, n] (or [n])."""
    W = np.ascontiguousarray(W, dtype=np.uint8)
    x = np.ascontiguousarray(x, dtype=np.float32)
    x2 = x.reshape(1, -1) if x.ndim == 1 else x
    batch = x2.shape[0]
    assert x2.shape[1] == k and W.size == n * row_bytes(wtype, k)
    y = np.empty((batch, n), dtype=np.float32)
    rc = lib().orc_matvec(wtype, scheme, _p(W), _p(x2), _p(y), n, k, batch, nthreads or max_threads())
    if rc != 0:
        raise ValueError("orc_matvec failed")
    return y[0] if x.ndim == 1 else y


def matvec_f64(wtype: int, W: np.ndarray, x: np.ndarray, n: int, k: int, nthreads: int = 0) -> np.ndarray:
    W = np.ascontiguousarray(W, dtype=np.uint8)
    x = np.ascontiguousarray(x, dtype=np.float32)
    x2 = x.reshape(1, -1) if x.ndim == 1 else x
    batch = x2.shape[0]
    y = np.empty((batch, n), dtype=np.float64)
    rc = lib().orc_matvec_f64(wtype, _p(W), _p(x2), _p(y), n, k, batch, nthreads or max_threads())
    if rc != 0:
        raise ValueError("orc_matvec_f64 failed")
    return y[0] if x.ndim == 1 else y


def prefill(wtype: int, W: np.ndarray, X_f16: np.ndarray, n: int, k: int, nthreads: int = 0) -> np.ndarray:
    """W uint8 [n, row_bytes]; X float16 [m, k]; returns fp32 [m, n]."""
    W = np.ascontiguousarray(W, dtype=np.uint8)
    X = np.ascontiguousarray(X_f16, dtype=np.float16)
    m = X.shape[0]
    assert X.shape[1] == k
    Y = np.empty((m, n), dtype=np.float32)
    rc = lib().orc_prefill(wtype, _p(W), _p(X.view(np.uint16)), _p(Y), m, n, k, nthreads or max_threads())
    if rc != 0:
        raise ValueError("orc_prefill failed")
    return Y
