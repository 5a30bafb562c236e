"""Quantized prefill matmul benchmark: Q4_0 / Q8_0 (default) or Q4_K / Q5_K / Q6_K weights 4096->14336 and 14336->4096, fp16
activations for M = 64, 512, 2048 tokens (seeded N(0,0.02) weights quantized on the host).

    python -m openagents_amd.prefill [--iters 20] [--formats q4_0,q8_0] [--m 64,512,2048] [--shapes 14336x4096,4096x14336]

Prints one JSON record per (format, shape, M): microseconds, TFLOP/s, GB/s and the fraction of the
roofline that binds (fp16 MFMA 2.5 PFLOP/s, or HBM 8 TB/s when the arithmetic intensity is below
the ridge of 312.5 FLOP/B).  Weight copies rotate so that the HBM-bound cases stream from memory.

With --sample-clock S every cell is additionally run back to back for S seconds while a thread reads the
shader clock from `rocm-smi --showclocks` five times a second; the record then carries the median clock
under that load and the fraction of the MFMA rate at that clock (2.5 PFLOP/s is quoted at 2.4 GHz, and the
device lowers its clock under sustained matrix work on real data).

With --compare-plans every cell is also timed under each explicit (tile_m, tile_n, ksplit, family) plan that accepts
the shape; the record then names the fastest of them beside the planner's default, which is how the planner's cost
model is checked.
"""
from __future__ import annotations

import argparse
import json
import re
import subprocess
import sys
import threading
import time

import numpy as np

from . import quantize
from ._ffi import Q4_0, Q4_K, Q5_K, Q6_K, Q8_0
from .backend import HipBackend, PsnError, prefill_plan, row_bytes

# (tile_m, tile_n, ksplit, family): the explicit plans --compare-plans tries (family 4 = four waves, 16 = producer / consumer,
# 32 = wide, 64 = weight-streaming for M <= 64, 128 = dense)
EXPLICIT_PLANS = [(64, 64, 1, 64), (64, 64, 2, 64), (64, 64, 4, 64), (64, 64, 8, 64),
                  (64, 64, 2, 4), (64, 64, 4, 4), (64, 64, 8, 4), (64, 128, 2, 4), (64, 128, 4, 4), (64, 128, 8, 4), (256, 128, 2, 4), (256, 128, 4, 4), (256, 128, 8, 4),
                  (128, 128, 1, 4), (256, 128, 1, 4), (256, 256, 1, 4), (256, 256, 2, 4), (256, 256, 4, 4),
                  (128, 128, 1, 16), (128, 128, 2, 16), (128, 128, 4, 16), (128, 128, 8, 16),
                  (128, 256, 1, 16), (128, 256, 2, 16), (128, 256, 4, 16), (128, 256, 8, 16),
                  (256, 256, 1, 32), (256, 256, 2, 32), (256, 256, 4, 32), (256, 256, 1, 128), (256, 256, 2, 128), (256, 256, 4, 128), (128, 256, 1, 128), (128, 256, 2, 128), (128, 256, 4, 128)]
MFMA_PEAK_TFLOPS = 2500.0
MFMA_PEAK_CLOCK_MHZ = 2400.0
HBM_PEAK_GBS = 8000.0


class ClockSampler:
    """Reads the current shader clock (MHz) from rocm-smi in a thread until stopped."""

    def __init__(self, period_s: float = 0.2):
        self.period, self.samples, self._stop = period_s, [], threading.Event()
        self._thread = threading.Thread(target=self._run, daemon=True)

    def _run(self):
        while not self._stop.is_set():
            try:
                out = subprocess.run(["rocm-smi", "--showclocks"], capture_output=True, text=True, timeout=5).stdout
                m = re.search(r"sclk clock level[^\n]*\((\d+)Mhz\)", out)
                if m:
                    self.samples.append(int(m.group(1)))
            except (OSError, subprocess.SubprocessError):
                pass
            self._stop.wait(self.period)

    def __enter__(self):
        self._thread.start()
        return self

    def __exit__(self, *exc):
        self._stop.set()
        self._thread.join()

    def median(self):
        s = sorted(self.samples[1:] or self.samples)          # the first sample may predate the ramp
        return s[len(s) // 2] if s else None


def main(argv=None):
    ap = argparse.ArgumentParser()
    ap.add_argument("--iters", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--formats", default="q4_0,q8_0")
    ap.add_argument("--m", default="64,512,2048")
    ap.add_argument("--seed", type=int, default=7)
    ap.add_argument("--sample-clock", type=float, default=0.0, metavar="S", help="also run each cell for S seconds and report the shader clock under that load")
    ap.add_argument("--shapes", default="14336x4096,4096x14336", help="weight shapes as NxK, comma separated")
    ap.add_argument("--compare-plans", action="store_true", help="also time every explicit plan and name the fastest")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run four 256 MiB device-to-device copies: a transfer of known size that hardware-counter runs scale FETCH_SIZE / WRITE_SIZE by")
    args = ap.parse_args(argv)
    fmts = {"q4_0": (Q4_0, quantize.quantize_q4_0), "q8_0": (Q8_0, quantize.quantize_q8_0), "q4_K": (Q4_K, quantize.quantize_q4_K),
            "q5_K": (Q5_K, quantize.quantize_q5_K), "q6_K": (Q6_K, quantize.quantize_q6_K)}
    be = HipBackend(0)
    rng = np.random.default_rng(args.seed)
    if args.calibrate_copy:
        nbytes = 256 << 20
        src, dst = be.alloc(nbytes), be.alloc(nbytes)
        for _ in range(4):
            be.copy(dst, src, nbytes)
        be.sync()
        src.free()
        dst.free()
    for fname in args.formats.split(","):
        qt, quant = fmts[fname]
        for n, k in (tuple(int(v) for v in t.split("x")) for t in args.shapes.split(",")):
            blocks = quant(rng.standard_normal((n, k), dtype=np.float32) * np.float32(0.02))
            copies = max(2, int(300e6 // blocks.nbytes) + 1)
            ws = [be.upload_weight(qt, blocks, n, k) for _ in range(copies)]
            for m in (int(v) for v in args.m.split(",")):
                x = be.upload(rng.standard_normal((m, k), dtype=np.float32).astype(np.float16))
                y = be.alloc(m * n * 4)
                def timed(tile=None):
                    for i in range(args.warmup):
                        be.quantized_matmul(ws[i % copies], x, y, m, tile)
                    be.sync()
                    e0, e1 = be.event(), be.event()
                    be.record(e0)
                    for i in range(args.iters):
                        be.quantized_matmul(ws[i % copies], x, y, m, tile)
                    be.record(e1)
                    t = be.elapsed_us(e0, e1) / args.iters
                    be.destroy_event(e0)
                    be.destroy_event(e1)
                    return t

                us = timed()
                compared = {}
                if args.compare_plans:
                    tried = []
                    for tile in EXPLICIT_PLANS:
                        try:
                            tried.append((timed(tile), tile))
                        except PsnError:                         # this plan does not take this shape or format
                            continue
                    if tried:
                        bt, bp = min(tried)
                        for _ in range(2):                       # the two contenders again, alternating, under the same clocks
                            bt, us = min(bt, timed(bp)), min(us, timed())
                        compared = {"best_explicit_plan": list(bp), "best_explicit_us": round(bt, 1), "default_over_best": round(us / bt, 3)}
                flops = 2.0 * m * n * k
                nbytes = n * row_bytes(qt, k) + m * k * 2 + m * n * 4
                tflops, gbs = flops / us / 1e6, nbytes / us / 1e3
                bound = "mfma" if flops / nbytes >= MFMA_PEAK_TFLOPS * 1e3 / HBM_PEAK_GBS else "hbm"
                frac = tflops / MFMA_PEAK_TFLOPS if bound == "mfma" else gbs / HBM_PEAK_GBS
                tm, tn, sp, wv = prefill_plan(m, n, k, be.compute_units, qt)
                sustained = {}
                if args.sample_clock > 0:
                    with ClockSampler() as cs:
                        t0, launches = time.time(), 0
                        s0, s1 = be.event(), be.event()
                        be.record(s0)
                        while time.time() - t0 < args.sample_clock:
                            for i in range(16):
                                be.quantized_matmul(ws[i % copies], x, y, m)
                            be.sync()
                            launches += 16
                        be.record(s1)
                        sus_us = be.elapsed_us(s0, s1) / launches
                        be.destroy_event(s0)
                        be.destroy_event(s1)
                    mhz = cs.median()
                    sustained = {"sustained_us": round(sus_us, 1), "sustained_TFLOPs": round(flops / sus_us / 1e6, 1), "sclk_MHz_under_load": mhz}
                    if mhz and bound == "mfma":
                        sustained["frac_of_mfma_rate_at_that_clock"] = round(flops / sus_us / 1e6 / (MFMA_PEAK_TFLOPS * mhz / MFMA_PEAK_CLOCK_MHZ), 4)
                print(json.dumps({"op": "quantized prefill matmul", "format": fname, "M": m, "N": n, "K": k, "us": round(us, 1),
                                  "TFLOPs": round(tflops, 1), "GBps": round(gbs, 1), "bound": bound, "frac_of_roofline": round(frac, 4),
                                  "kernel": {64: f"psn_prefill_{fname}_skinny", 32: f"psn_prefill_{fname}_wide", 128: f"psn_prefill_{fname}_unpack + psn_prefill_dense_f16" + ("_m128" if tm == 128 else "")}.get(wv, f"psn_prefill_{fname}_m{tm}_n{tn}" + {4: "", 16: "_ws"}.get(wv, "")),
                                  "ksplit": sp, "iters": args.iters, **sustained, **compared}), flush=True)
            for w in ws:
                w.buf.free()
    return 0


if __name__ == "__main__":
    sys.exit(main())
