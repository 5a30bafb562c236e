#!/usr/bin/env python3
"""Headline benchmark: Q4_0 decode matvec over the Llama-3-8B projection shapes at batch 1.

A "step" is one token's worth of projection matvecs: 32 layers x (q, k, v | o | gate, up | down),
fp32 activations in, fp32 out, activation scheme Q8 (x quantized to Q8_0 blocks, int8 dot, fp16
block scales applied in fp32).  Matrices that share their input go out as one launch (q/k/v and
gate/up), so a step is 128 launches replayed from one HIP graph; every layer has its own weight
buffers (3.93 GB per step), which defeats the 256 MB Infinity Cache.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--cpu-seconds S]

Prints ONE JSON line.  `value` is whole-step algorithmic GB/s with everything resident in HBM
before the timed region; `roofline` is the dominant kernel's achieved HBM bandwidth measured with
HIP events on the launch stream; `cpu_baseline` is the CPU oracle timed on this host's cores on a
bounded sample of the same workload (a reported baseline, not the target).  `records` carries the
other configurations of the metric -- Q8_0 4096x4096, Q4_K at batch 1/2/4/8, the twelve prefill
cells, the 8B-shaped decode step -- one throughput record each (openagents_amd/records.py), and
`read_calibration` what a kernel that only reads reaches at the four launch sizes.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0
# HBM bytes per launch from hardware counters, not measured by this run: rocprofv3 --pmc FETCH_SIZE and
# --pmc WRITE_SIZE over this same command (two runs), each scaled by what the same counter reads for a
# 256 MiB device-to-device copy (x1.99979 and x1.0000; the copies are what --calibrate-copy adds).  The
# figures and the commands are in profiles/matvec_q4_0_llama3_8b_step.md.
MEASURED_TRAFFIC_BYTES = {"qkv": 14_517_000, "o": 9_781_300, "gate_up": 66_512_700, "down": 33_708_900}
TRAFFIC_SOURCE = "profiles/matvec_q4_0_llama3_8b_step.md (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE, copy-calibrated)"
HIDDEN, KV, FFN, LAYERS = 4096, 1024, 14336, 32
BPW_Q4_0 = 18.0 / 32.0


def algo_bytes(ns, k, batch=1):
    """Algorithmic bytes of one launch: GGUF weight bytes + fp32 x in + fp32 y out."""
    return sum(n * k * BPW_Q4_0 + batch * n * 4 for n in ns) + batch * k * 4


# the four launches of a layer: (name, output rows of the matrices sharing the launch, K)
LAUNCHES = [("qkv", [HIDDEN, KV, KV], HIDDEN), ("o", [HIDDEN], HIDDEN),
            ("gate_up", [FFN, FFN], HIDDEN), ("down", [HIDDEN], FFN)]


def cpu_model():
    try:
        with open("/proc/cpuinfo") as f:
            for line in f:
                if line.startswith("model name"):
                    return line.split(":", 1)[1].strip()
    except OSError:
        pass
    return "unknown"


def make_layer(seed):
    """One layer's seeded N(0, 0.02) weights, quantized to Q4_0 by the host quantizer."""
    from openagents_amd import quantize
    rng = np.random.default_rng(seed)
    out = {}
    for name, ns, k in LAUNCHES:
        out[name] = [quantize.quantize_q4_0((rng.standard_normal((n, k), dtype=np.float32) * np.float32(0.02))) for n in ns]
    return out


def main(argv=None):
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--layers", type=int, default=LAYERS, help="weight copies a step walks through")
    ap.add_argument("--cpu-seconds", type=float, default=10.0, help="budget of the CPU baseline leg (0 skips it)")
    ap.add_argument("--seed", type=int, default=1234)
    ap.add_argument("--calibrate-copy", action="store_true", help="also run four 256 MiB device-to-device copies (counter calibration)")
    ap.add_argument("--no-records", action="store_true", help="headline only: skip the records of the other configurations")
    ap.add_argument("--record-samples", type=int, default=7)
    args = ap.parse_args(argv)
    if args.gpus != 1:
        print("bench.py: this build drives one GPU; --gpus N with N > 1 is not supported "
              "(the path would shard by weight rows across GPUs, but nothing here launches a second rank)", file=sys.stderr)
        return 2

    from openagents_amd import _ffi
    from openagents_amd.backend import HipBackend, matvec_plan

    be = HipBackend(0)
    be.reserve_prefill(14336, 4096)      # workspace of the dense prefill family (config 4 records), sized before any graph is captured
    t_setup = time.time()
    layer = make_layer(args.seed)
    rng = np.random.default_rng(args.seed + 1)
    x_host = {"qkv": rng.standard_normal(HIDDEN, dtype=np.float32), "o": rng.standard_normal(HIDDEN, dtype=np.float32),
              "gate_up": rng.standard_normal(HIDDEN, dtype=np.float32), "down": rng.standard_normal(FFN, dtype=np.float32)}
    # every layer gets its own device copies of the same bytes: distinct addresses, 3.93 GB in all
    weights = []
    for _ in range(args.layers):
        weights.append({name: [be.upload_weight(_ffi.Q4_0, blk, n, k) for blk, n in zip(layer[name], ns)]
                        for name, ns, k in LAUNCHES})
    xs = {name: be.upload(x_host[name]) for name, _, _ in LAUNCHES}
    ys = {name: [be.alloc(n * 4) for n in ns] for name, ns, _ in LAUNCHES}
    be.reserve(FFN, 1)
    be.sync()
    setup_s = time.time() - t_setup

    def capture(names):
        be.begin_capture()
        for lw in weights:
            for name, _, _ in LAUNCHES:
                if name in names:
                    be.quantized_matvec_multi(lw[name], xs[name], ys[name], 1, _ffi.ACT_Q8)
        return be.end_capture()

    def time_graph(graph, reps):
        e0, e1 = be.event(), be.event()
        be.record(e0)
        for _ in range(reps):
            be.launch_graph(graph)
        be.record(e1)
        us = be.elapsed_us(e0, e1)
        be.destroy_event(e0)
        be.destroy_event(e1)
        return us

    step_graph = capture({n for n, _, _ in LAUNCHES})
    bytes_per_step = args.layers * sum(algo_bytes(ns, k) for _, ns, k in LAUNCHES)

    # ---- the timed region: W warm-up steps, then exactly K steps between two synchronizations
    for _ in range(args.warmup):
        be.launch_graph(step_graph)
    be.sync()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        be.launch_graph(step_graph)
    be.sync()
    t1 = time.perf_counter()
    ms_per_step = (t1 - t0) * 1e3 / args.steps
    value = bytes_per_step / (ms_per_step * 1e-3) / 1e9

    # ---- the same 128 launches with no ordering between them, alternating over two streams (two graph
    # branches): what the kernels stream when the ramp of one launch can run under the tail of another.
    # Reported beside `value`, never as `value`: in a decoder the launches of a layer depend on each other.
    side = be.new_stream()
    be.begin_capture()
    main = be.stream
    be.stream_wait(side, main)                               # fork
    i = 0
    for lw in weights:
        for name, _, _ in LAUNCHES:
            if i % 2:
                with be.on_stream(side):
                    be.quantized_matvec_multi(lw[name], xs[name], ys[name], 1, _ffi.ACT_Q8)
            else:
                be.quantized_matvec_multi(lw[name], xs[name], ys[name], 1, _ffi.ACT_Q8)
            i += 1
    be.stream_wait(main, side)                               # join
    two_graph = be.end_capture()
    for _ in range(args.warmup):
        be.launch_graph(two_graph)
    be.sync()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        be.launch_graph(two_graph)
    be.sync()
    ms_two = (time.perf_counter() - t0) * 1e3 / args.steps
    be.destroy_graph(two_graph)

    # ---- per-launch figures with HIP events on the launch stream: one graph per launch kind
    per_launch = {}
    for name, ns, k in LAUNCHES:
        g = capture({name})
        time_graph(g, 2)
        us = time_graph(g, max(3, args.steps // 4)) / (max(3, args.steps // 4) * args.layers)
        per_launch[name] = {"us": round(us, 3), "algo_MB": round(algo_bytes(ns, k) / 1e6, 3),
                            "GBps": round(algo_bytes(ns, k) / us / 1e3, 1)}
        be.destroy_graph(g)

    # dominant kernel: group the launch kinds by the kernel the library picks for them and take the
    # group a step spends most time in; its figures are averages over that group's launches
    def kernel_of(ns, k):
        p = matvec_plan(_ffi.Q4_0, _ffi.ACT_Q8, sum(ns), k, 1, be.compute_units, True)
        if p.stream:
            return f"psn_mvs_q4_0_q8_g{p.lanes_per_row}" + {1: "_lds", 2: "_xf"}[p.stage_lds] + f"_s{len(ns)}"
        return f"psn_mv_q4_0_q8_g{p.lanes_per_row}_r{p.rows_in_flight}_b{p.batch_tile}" + {0: "", 1: "_lds", 2: "_xf"}[p.stage_lds]
    groups = {}
    for name, ns, k in LAUNCHES:
        groups.setdefault(kernel_of(ns, k), []).append(name)
    dom_kernel = max(groups, key=lambda kn: sum(per_launch[n]["us"] for n in groups[kn]))
    dom_names = groups[dom_kernel]
    g = capture(set(dom_names))
    time_graph(g, 2)
    reps = max(3, args.steps // 4)
    dom_us = time_graph(g, reps) / (reps * args.layers * len(dom_names))
    be.destroy_graph(g)
    dom_bytes = sum(algo_bytes(ns, k) for name, ns, k in LAUNCHES if name in dom_names) / len(dom_names)
    achieved = dom_bytes / dom_us / 1e3
    roofline = {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                "frac": round(achieved / HBM_PEAK_GBS, 4),
                "traffic": int(sum(MEASURED_TRAFFIC_BYTES[n] for n in dom_names) / len(dom_names)), "traffic_source": TRAFFIC_SOURCE,
                "kernel": dom_kernel,
                "avg_launch_us": round(dom_us, 3), "algo_bytes_per_launch": int(dom_bytes),
                "launches_per_step": args.layers * len(dom_names),
                "note": "average over the " + ", ".join(dom_names) + " launches, which share this kernel ("
                        + ", ".join(f"{per_launch[n]['algo_MB']} MB" for n in dom_names) + ")"}

    if args.calibrate_copy:
        # a plain device-to-device copy of known size, so hardware-counter runs can scale FETCH_SIZE /
        # WRITE_SIZE by what the same counters read for it
        nbytes = 256 << 20
        src, dst = be.alloc(nbytes), be.alloc(nbytes)
        for _ in range(4):
            be.copy(dst, src, nbytes)
        be.sync()

    # ---- parity spot check and CPU baseline (the oracle is the checker and the timed CPU path)
    cpu = None
    parity = None
    if args.cpu_seconds > 0:
        import oracle
        be.launch_graph(step_graph)
        be.sync()
        worst = 0.0
        for name, ns, k in LAUNCHES:
            for blk, n, y in zip(layer[name], ns, ys[name]):
                ref = oracle.matvec(oracle.Q4_0, oracle.ACT_Q8, blk, x_host[name], n, k)
                got = y.download(np.float32, (n,))
                worst = max(worst, float(np.max(np.abs(got - ref)) / np.max(np.abs(ref))))
        parity = {"metric": "max|y-ref|/max|ref| over all 7 projections vs CPU oracle, scheme Q8", "value": worst, "gate": 1e-3}
        layer_bytes = sum(algo_bytes([n], k) for _, ns, k in LAUNCHES for n in ns)

        def cpu_leg(threads, seconds):
            done, t_cpu0 = 0, time.perf_counter()
            while True:
                for name, ns, k in LAUNCHES:
                    for blk, n in zip(layer[name], ns):
                        oracle.matvec(oracle.Q4_0, oracle.ACT_Q8, blk, x_host[name], n, k, nthreads=threads)
                done += 1
                if time.perf_counter() - t_cpu0 >= seconds:
                    break
            cpu_s = time.perf_counter() - t_cpu0
            return done, cpu_s, round(done * layer_bytes / cpu_s / 1e9, 2)

        threads = oracle.max_threads()
        done1, s1, gbs1 = cpu_leg(1, args.cpu_seconds * 0.4)
        done, cpu_s, gbs = cpu_leg(threads, args.cpu_seconds * 0.6)
        cpu = {"value": gbs, "unit": "GB/s", "cores": threads, "kind": "port",
               "sample": f"{done} x one layer's 7 Q4_0 projections (same bytes and activations as the GPU run), "
                         f"{cpu_s:.1f} s, OpenMP over rows",
               "single_thread": {"value": gbs1, "unit": "GB/s", "cores": 1, "sample": f"{done1} x the same layer, {s1:.1f} s"},
               "host": {"nproc": os.cpu_count(), "usable_threads": threads, "cpu_model": cpu_model()},
               "provenance": "this build's C restatement of the CPU quantized path (oracle/), not Psionic's binary"}

    records, calibration = None, None
    if not args.no_records:
        from openagents_amd import records as R
        for lw in weights:                                   # the headline's 3.9 GB of copies are no longer needed
            for ts in lw.values():
                for t in ts:
                    t.buf.free()
        weights.clear()
        calibration = R.read_calibration(be, args.record_samples)
        shared = {(_ffi.Q4_0, FFN, HIDDEN): layer["gate_up"][0], (_ffi.Q4_0, HIDDEN, FFN): layer["down"][0]}
        records = (R.config1(be, args.record_samples, cpu=args.cpu_seconds > 0) + R.config3(be, args.record_samples)
                   + R.config4(be, args.record_samples, weights=shared) + R.config5(be, args.record_samples))

    out = {
        "metric": "quant matvec GB/s", "value": round(value, 1), "unit": "GB/s", "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "u4 x int8 -> int32, fp32 scales/accumulate",
        "data": "synthetic: seeded N(0,0.02) fp32 weights quantized to GGUF Q4_0 on the host (one layer, copied to "
                f"{args.layers} distinct device allocations); activations fp32 N(0,1)",
        "config": {"workload": "Q4_0 decode matvec, Llama-3-8B projections (4096->4096 q,o; 4096->1024 k,v; 4096->14336 gate,up; "
                               "14336->4096 down), batch 1, 32 layers per step, fp32 in/out, activation scheme Q8",
                   "launches_per_step": args.layers * len(LAUNCHES), "bytes_per_step": int(bytes_per_step),
                   "graph_replay": True},
        "frac_of_hbm_peak": round(value / HBM_PEAK_GBS, 4),
        "independent_launches_two_streams": {"ms_per_step": round(ms_two, 4), "GBps": round(bytes_per_step / (ms_two * 1e-3) / 1e9, 1),
                                             "note": "same launches without ordering between them, two graph branches; not the headline"},
        "matvec_tokens_per_s": round(1e3 / ms_per_step, 1),
        "per_launch": per_launch,
        "roofline": roofline,
        "cpu_baseline": cpu,
        "parity": parity,
        "read_calibration": calibration,
        "records": records,
        "device": {"arch": be.arch, "compute_units": be.compute_units}, "setup_s": round(setup_s, 1),
    }
    print(json.dumps(out))
    return 0


if __name__ == "__main__":
    sys.exit(main())
