#!/usr/bin/env python3
"""Writes tests/golden/psn_golden.npz: small seeded inputs and the outputs the CPU oracle gives for them.

    python tests/golden/make_fixtures.py

The reference tree holds no vector for this path, so these are the oracle's own outputs, frozen: a later
change to the oracle (or to a kernel) that moves any of these bytes shows up as a diff against data that
does not depend on the current oracle build.  Regenerate only after such a change has been understood.
Everything is plain numpy arrays (loaded with allow_pickle=False).
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

N, K, BATCH, M = 8, 512, 2, 4
NB = 32                                   # rows of the batch-8 fixtures
FORMATS = {"q4_0": 2, "q8_0": 8, "q4_K": 12, "q6_K": 14, "q5_K": 13}      # appended in this order: a format's seed is its position


def inputs(seed):
    rng = np.random.default_rng(seed)
    w = (rng.standard_normal((N, K), dtype=np.float32) * np.float32(0.02)).astype(np.float32)
    x = rng.standard_normal((BATCH, K), dtype=np.float32)
    xh = rng.standard_normal((M, K), dtype=np.float32).astype(np.float16)
    return w, x, xh


def build():
    import oracle
    out = {}
    for i, (name, t) in enumerate(FORMATS.items()):
        w, x, xh = inputs(7000 + i)
        blocks = oracle.quantize(t, w, nthreads=1)
        out[f"{name}_w"] = w
        out[f"{name}_x"] = x
        out[f"{name}_blocks"] = blocks
        out[f"{name}_deq"] = oracle.dequantize(t, blocks, K)
        out[f"{name}_y_q8"] = oracle.matvec(t, oracle.ACT_Q8, blocks, x, N, K, nthreads=1)
        out[f"{name}_y_f32"] = oracle.matvec(t, oracle.ACT_F32, blocks, x, N, K, nthreads=1)
        out[f"{name}_xh"] = xh
        out[f"{name}_y_prefill"] = oracle.prefill(t, blocks, xh, N, K, nthreads=1)
    # 32 rows x 8 activation columns: the shape class the small-batch (batch 2..8) kernels of Q4_K / Q5_K serve
    for i, name in enumerate(("q4_K", "q5_K")):
        rng = np.random.default_rng(7200 + i)
        w = rng.standard_normal((NB, K), dtype=np.float32) * np.float32(0.02)
        x = rng.standard_normal((8, K), dtype=np.float32)
        blocks = oracle.quantize(FORMATS[name], w, nthreads=1)
        out[f"batch8_{name}_blocks"] = blocks
        out[f"batch8_{name}_x"] = x
        out[f"batch8_{name}_y_q8"] = oracle.matvec(FORMATS[name], oracle.ACT_Q8, blocks, x, NB, K, nthreads=1)
    _, x, _ = inputs(7100)
    out["act_x"] = x
    out["act_q8_0"] = oracle.quantize(oracle.Q8_0, x, nthreads=1)
    out["act_q8_K"] = oracle.quantize(oracle.Q8_K, x, nthreads=1)
    return out


if __name__ == "__main__":
    path = os.path.join(HERE, "psn_golden.npz")
    np.savez_compressed(path, **build())
    print("wrote", path, os.path.getsize(path), "bytes")
