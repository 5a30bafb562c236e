#!/usr/bin/env python3
"""Headline benchmark: Q4_0 decode matvec over the Llama-3-8B projection shapes at batch 1.

A "step" is one token's worth of projection matvecs: 32 layers x (q, k, v | o | gate, up | down),
fp32 activations in, fp32 out, activation scheme Q8 (x quantized to Q8_0 blocks, int8 dot, fp16
block scales applied in fp32).  Matrices that share their input go out as one launch (q/k/v and
gate/up), so a step is 128 launches replayed from one HIP graph; every layer has its own weight
buffers (3.93 GB per step), which defeats the 256 MB Infinity Cache.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--cpu-seconds S] [--records-out FILE]

The LAST line of stdout is ONE JSON object of fewer than 2000 characters: the headline (`value` is whole-step
algorithmic GB/s with everything resident in HBM before the timed region), `roofline` (the dominant kernel's
achieved HBM bandwidth, measured with HIP events on the launch stream), `cpu_baseline` (the CPU oracle timed on
this host's cores on a bounded sample of the same workload: a reported baseline, not the target), the parity of
the run against the oracle, and `configs`, one figure per other configuration of the metric (fraction of the
roofline that bounds it).  Everything else -- one throughput record per configuration with its own parity
verdict (openagents_amd/records.py), the per-launch table, the read-only calibration -- goes to the file named
by --records-out (default gpurun_out/bench_records.json), not to stdout.
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
MAX_LINE_CHARS = 2000
# HBM bytes per launch from hardware counters, not measured by this run: rocprofv3 --pmc FETCH_SIZE and
# --pmc WRITE_SIZE over this same command (two runs), each scaled by what the same counter reads for a
# 256 MiB device-to-device copy (the copies are what --calibrate-copy adds).  Keyed by the kernel the figure was
# taken on: when the library picks another kernel for the launch, `traffic` is null instead of a stale number.
# The figures and the commands are in profiles/matvec_q4_0_llama3_8b_step.md.
MEASURED_TRAFFIC_BYTES = {"psn_mvs_q4_0_q8_g16_xf_s2": 66_491_100, "psn_mvs_q4_0_q8_g16_xf_s3": 14_512_800,
                          "psn_mvs_q4_0_q8_g16_xf_s1": 9_782_300, "psn_mvs_q4_0_q8_g64_xf_s1": 33_703_700}
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


class OracleChecker:
    """The parity checker handed to the record builders: the CPU oracle on the record's own bytes.  Lives here,
    outside the package, because the package must never touch the oracle."""

    def __init__(self):
        import oracle
        self.orc = oracle
        self.max_threads = oracle.max_threads()

    def matvec(self, qtype, blocks, x, n, k):
        return self.orc.matvec(qtype, self.orc.ACT_Q8, blocks, x, n, k)

    def prefill(self, qtype, blocks, x_f16, n, k):
        return self.orc.prefill(qtype, blocks, x_f16, n, k)

    def __call__(self, qtype, blocks, x, n, k, threads):
        """The timed CPU path of the config-1 record."""
        return self.orc.matvec(qtype, self.orc.ACT_Q8, blocks, x, n, k, nthreads=threads)

    def decode_last_layer(self, shape, protos, got):
        """Teacher-forced reference of the launches that end a step, from the device's own vectors: gate | up (or, where
        the device applied SwiGLU inside that launch, silu(gate) * up and the down projection of the device's own
        `act`) from the residual `x` that entered the last layer's FFN norm, the logits from x + down (norm weights 1)."""
        sys.path.insert(0, os.path.join(ROOT, "tests"))
        from decoderef import rmsnorm_ref
        orc, s = self.orc, shape
        n_unique = sum(1 for name in protos if name.endswith(".wq"))
        p = f"layer{(s.n_layers - 1) % n_unique}."
        ones, eps = np.ones(s.hidden, np.float32), np.float32(s.eps)
        xn = rmsnorm_ref(got["x"], ones, eps)
        out = {"gate": orc.matvec(orc.Q4_K, orc.ACT_Q8, protos[p + "w_gate"], xn, s.ffn, s.hidden).reshape(-1),
               "up": orc.matvec(orc.Q4_K, orc.ACT_Q8, protos[p + "w_up"], xn, s.ffn, s.hidden).reshape(-1)}
        if "act" in got:
            # SwiGLU ran inside the gate | up launch: its output, and the down projection of the device's own output
            g, u = out["gate"].astype(np.float64), out["up"].astype(np.float64)
            out["act"] = (g / (1.0 + np.exp(-g)) * u).astype(np.float32)
            out["down"] = orc.matvec(orc.Q4_K, orc.ACT_Q8, protos[p + "w_down"], got["act"], s.hidden, s.ffn).reshape(-1)
        uniq = protos["lm_head"].shape[0]
        xf = rmsnorm_ref((got["x"] + got["down"]).astype(np.float32), ones, eps)
        head = orc.matvec(orc.Q6_K, orc.ACT_Q8, protos["lm_head"], xf, uniq, s.hidden).reshape(-1)
        out["logits"] = np.tile(head, -(-s.vocab // uniq))[:s.vocab]
        return out

    def decode_step(self, shape, protos, x0, kv, pos):
        """Logits of one token at position `pos` of the synthetic model whose layers all hold the matrices in
        `protos` (norm weights 1, LM head = `lm_head` rows tiled to the vocabulary), every layer's K and V cache
        pre-filled with `kv` [pos, kv_dim] fp16: float64 numpy around the oracle's matvecs."""
        sys.path.insert(0, os.path.join(ROOT, "tests"))
        from decoderef import attention_ref, rmsnorm_ref, rope_ref
        orc, s = self.orc, shape
        eps = np.float32(s.eps)
        ones = np.ones(s.hidden, np.float32)

        def mv(name, vec, n, k, qtype=None):
            return orc.matvec(qtype or orc.Q4_K, orc.ACT_Q8, protos[name], vec, n, k).reshape(-1)

        x = x0.astype(np.float32).copy()
        cache_k = np.zeros((pos + 1, s.kv_dim), np.float16)
        cache_v = np.zeros((pos + 1, s.kv_dim), np.float16)
        n_unique = sum(1 for name in protos if name.endswith(".wq"))
        for li in range(s.n_layers):
            p = f"layer{li % n_unique}."
            xn = rmsnorm_ref(x, ones, eps)
            q = rope_ref(mv(p + "wq", xn, s.hidden, s.hidden), s.n_heads, s.head_dim, pos, s.rope_theta)
            kk = rope_ref(mv(p + "wk", xn, s.kv_dim, s.hidden), s.n_kv_heads, s.head_dim, pos, s.rope_theta)
            vv = mv(p + "wv", xn, s.kv_dim, s.hidden)
            cache_k[:pos], cache_v[:pos] = kv, kv
            cache_k[pos], cache_v[pos] = kk.astype(np.float16), vv.astype(np.float16)
            att = attention_ref(q, cache_k, cache_v, s.n_heads, s.n_kv_heads, s.head_dim, pos + 1)
            x = x + mv(p + "wo", att, s.hidden, s.hidden)
            xn = rmsnorm_ref(x, ones, eps)
            g, u = mv(p + "w_gate", xn, s.ffn, s.hidden), mv(p + "w_up", xn, s.ffn, s.hidden)
            g64 = g.astype(np.float64)
            act = (g64 / (1 + np.exp(-g64)) * u).astype(np.float32)
            x = x + mv(p + "w_down", act, s.hidden, s.ffn)
        uniq = protos["lm_head"].shape[0]
        head = mv("lm_head", rmsnorm_ref(x, ones, eps), uniq, s.hidden, orc.Q6_K)
        return np.tile(head, -(-s.vocab // uniq))[:s.vocab]


def compact_configs(records):
    """One figure per configuration for the headline line: fraction of the roofline that bounds it."""
    out = {"c1_q8_0_4096": None, "c3_q4_K_b1248": {}, "c4_m64_512_2048": {}, "c5": None}
    bad, lm_head = 0, None
    for r in records or []:
        op, frac = r["opRef"], r["roofline"]["fraction"]
        bad += r["parity"]["status"] != "pass"
        parts = op.split(".")
        if op.startswith("matvec.q8_0"):
            out["c1_q8_0_4096"] = frac
        elif op.startswith("matvec.q4_K"):
            out["c3_q4_K_b1248"].setdefault(parts[2], []).append(frac)
        elif op.startswith("prefill."):
            out["c4_m64_512_2048"].setdefault(parts[1] + "." + parts[2], []).append(frac)
        elif op.startswith("matvec.q6_K"):
            lm_head = frac
        elif op.startswith("decode.step"):
            out["c5"] = {"tok_s": r["tokensPerSecond"], "matvec_share": r.get("matvec_share"), "matvec_frac": frac}
    if lm_head is not None and out["c5"] is not None:
        out["c5"]["lm_head_q6_K_frac"] = lm_head
    out["parity_not_pass"] = bad
    return out


def assemble_line(head: dict, records, records_file) -> str:
    """The one JSON line the driver parses: headline fields, roofline, cpu_baseline, parity, a compact summary of
    the other configurations.  Long texts are cut rather than letting the line pass MAX_LINE_CHARS."""
    roof = head["roofline"]
    cpu = head.get("cpu_baseline")
    line = {
        "metric": "quant matvec GB/s", "value": head["value"], "unit": "GB/s", "n_gpus": 1, "steps": head["steps"], "warmup": head["warmup"],
        "ms_per_step": head["ms_per_step"], "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "int8",
        "data": "synthetic",
        "config": {"workload": "Q4_0 decode matvec, Llama-3-8B projections (q,o 4096x4096; k,v 4096->1024; gate,up 4096->14336; "
                               "down 14336->4096), batch 1, 32 layers/step, fp32 in/out, act scheme Q8, seeded N(0,0.02) weights",
                   "launches_per_step": head["launches_per_step"], "bytes_per_step": head["bytes_per_step"], "graph_replay": True},
        "frac_of_hbm_peak": round(head["value"] / HBM_PEAK_GBS, 4),
        "roofline": {k: roof[k] for k in ("bound", "achieved", "peak", "unit", "frac", "traffic", "kernel", "avg_launch_us", "algo_bytes_per_launch")},
        "cpu_baseline": None if cpu is None else {"value": cpu["value"], "unit": cpu["unit"], "cores": cpu["cores"], "kind": cpu["kind"],
                                                  "sample": cpu["sample"][:120], "single_thread": cpu["single_thread"]["value"]},
        "parity": head.get("parity"),
        "per_launch_us": head.get("per_launch_us"),
        "two_streams_GBps": head.get("two_streams_GBps"),
        "configs": compact_configs(records) if records else None,
        "records_file": records_file,
    }
    text = json.dumps(line, separators=(",", ":"))
    if len(text) >= MAX_LINE_CHARS:                      # never happens with the fields above; a guard, not a code path to rely on
        line["configs"] = None
        line["config"]["workload"] = line["config"]["workload"][:80]
        text = json.dumps(line, separators=(",", ":"))
    return text


def main(argv=None):
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--layers", type=int, default=LAYERS, help="weight copies a step walks through")
    ap.add_argument("--cpu-seconds", type=float, default=10.0, help="budget of the CPU baseline leg (0 skips it and every parity check)")
    ap.add_argument("--seed", type=int, default=1234)
    ap.add_argument("--calibrate-copy", action="store_true", help="also run four 256 MiB device-to-device copies (counter calibration)")
    ap.add_argument("--no-records", action="store_true", help="headline only: skip the records of the other configurations")
    ap.add_argument("--record-samples", type=int, default=21)
    ap.add_argument("--records-out", default=os.path.join("gpurun_out", "bench_records.json"),
                    help="file that receives the full records, the per-launch table and the calibration")
    ap.add_argument("--vendor-gemm", action="store_true",
                    help="also time the vendor library's fp16 GEMM (torch.matmul) at the prefill shapes: a calibration of what "
                         "fp16 MFMA sustains on this device, written to the records file; runs in a child process of its own "
                         "(torch brings its own HIP runtime) before this one touches the GPU")
    ap.add_argument("--vendor-gemm-only", action="store_true", help=argparse.SUPPRESS)
    args = ap.parse_args(argv)
    if args.vendor_gemm_only:
        print(json.dumps(vendor_gemm_calibration()))
        return 0
    vendor = None
    if args.vendor_gemm:
        import subprocess
        p = subprocess.run([sys.executable, os.path.abspath(__file__), "--vendor-gemm-only"], capture_output=True, text=True, timeout=600)
        try:
            vendor = json.loads(p.stdout.strip().splitlines()[-1])
        except (IndexError, ValueError):
            vendor = {"error": (p.stderr or p.stdout)[-400:]}
    if args.gpus != 1:
        print("bench.py: this build drives one GPU; --gpus N with N > 1 is not supported "
              "(the path would shard by weight rows across GPUs, but nothing here launches a second rank)", file=sys.stderr)
        return 2

    from openagents_amd import _ffi
    from openagents_amd import records as R
    from openagents_amd.backend import HipBackend

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
    main_stream = be.stream
    be.stream_wait(side, main_stream)                        # fork
    i = 0
    for lw in weights:
        for name, _, _ in LAUNCHES:
            if i % 2:
                with be.on_stream(side):
                    be.quantized_matvec_multi(lw[name], xs[name], ys[name], 1, _ffi.ACT_Q8)
            else:
                be.quantized_matvec_multi(lw[name], xs[name], ys[name], 1, _ffi.ACT_Q8)
            i += 1
    be.stream_wait(main_stream, side)                        # join
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

    # ---- per-launch figures with HIP events on the launch stream: one graph per launch kind; the kernel of each
    # kind is read back from the library's launch log
    per_launch, kernel_of = {}, {}
    for name, ns, k in LAUNCHES:
        kernel_of[name] = R.launched_kernels(be, lambda: be.quantized_matvec_multi(weights[0][name], xs[name], ys[name], 1, _ffi.ACT_Q8))
        g = capture({name})
        time_graph(g, 2)
        us = time_graph(g, max(3, args.steps // 4)) / (max(3, args.steps // 4) * args.layers)
        per_launch[name] = {"us": round(us, 3), "algo_MB": round(algo_bytes(ns, k) / 1e6, 3),
                            "GBps": round(algo_bytes(ns, k) / us / 1e3, 1), "kernel": kernel_of[name]}
        be.destroy_graph(g)

    # dominant kernel: group the launch kinds by the kernel the library ran for them and take the
    # group a step spends most time in; its figures are averages over that group's launches
    groups = {}
    for name, _, _ in LAUNCHES:
        groups.setdefault(kernel_of[name], []).append(name)
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
                "traffic": MEASURED_TRAFFIC_BYTES.get(dom_kernel) if len(dom_names) == 1 else None,
                "traffic_source": "profiles/matvec_q4_0_llama3_8b_step.md (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE, copy-calibrated)",
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
    cpu, parity, checker = None, None, None
    if args.cpu_seconds > 0:
        checker = OracleChecker()
        oracle = checker.orc
        be.launch_graph(step_graph)
        be.sync()
        worst = 0.0
        for name, ns, k in LAUNCHES:
            for blk, n, y in zip(layer[name], ns, ys[name]):
                ref = oracle.matvec(oracle.Q4_0, oracle.ACT_Q8, blk, x_host[name], n, k)
                got = y.download(np.float32, (n,))
                worst = max(worst, float(np.max(np.abs(got - ref)) / np.max(np.abs(ref))))
        parity = {"metric": "max|y-ref|/max|ref| over all 7 projections vs CPU oracle, scheme Q8", "value": worst, "gate": 1e-3,
                  "status": "pass" if worst < 1e-3 else "fail"}
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
               "sample": f"{done} x one layer's 7 Q4_0 projections (same bytes as the GPU run), {cpu_s:.1f} s, OpenMP over rows",
               "single_thread": {"value": gbs1, "unit": "GB/s", "cores": 1, "sample": f"{done1} x the same layer, {s1:.1f} s"},
               "host": {"nproc": os.cpu_count(), "usable_threads": threads, "cpu_model": cpu_model()},
               "provenance": "this build's C restatement of the CPU quantized path (oracle/), not Psionic's binary"}

    records, calibration = None, None
    if not args.no_records:
        for lw in weights:                                   # the headline's 3.9 GB of copies are no longer needed
            for ts in lw.values():
                for t in ts:
                    t.buf.free()
        weights.clear()
        calibration = R.read_calibration(be, args.record_samples)
        shared = {(_ffi.Q4_0, FFN, HIDDEN): layer["gate_up"][0], (_ffi.Q4_0, HIDDEN, FFN): layer["down"][0]}
        records = (R.config1(be, args.record_samples, checker=checker, cpu_path=checker) + R.config3(be, args.record_samples, checker=checker)
                   + R.config4(be, args.record_samples, weights=shared, checker=checker) + R.config5(be, args.record_samples, checker=checker))
    head = {"value": round(value, 1), "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms_per_step, 4),
            "launches_per_step": args.layers * len(LAUNCHES), "bytes_per_step": int(bytes_per_step), "roofline": roofline,
            "cpu_baseline": cpu, "parity": None if parity is None else {"value": float(f"{parity['value']:.3e}"), "gate": 1e-3, "status": parity["status"]},
            "per_launch_us": {n: per_launch[n]["us"] for n in per_launch},
            "two_streams_GBps": round(bytes_per_step / (ms_two * 1e-3) / 1e9, 1)}
    full = {"headline": head, "parity": parity, "per_launch": per_launch,
            "independent_launches_two_streams": {"ms_per_step": round(ms_two, 4), "GBps": head["two_streams_GBps"],
                                                 "note": "same launches without ordering between them, two graph branches; not the headline"},
            "matvec_tokens_per_s": round(1e3 / ms_per_step, 1),
            "data": "synthetic: seeded N(0,0.02) fp32 weights quantized to GGUF Q4_0 on the host (one layer, copied to "
                    f"{args.layers} distinct device allocations); activations fp32 N(0,1)",
            "dtype": "u4 x int8 -> int32, fp32 scales/accumulate",
            "read_calibration": calibration, "vendor_gemm_calibration": vendor, "records": records,
            "health": R.health(be), "worker_attachment": R.worker_attachment(records) if records else None,
            "device": {"arch": be.arch, "compute_units": be.compute_units}, "setup_s": round(setup_s, 1)}
    records_file = None
    try:
        d = os.path.dirname(args.records_out)
        if d:
            os.makedirs(d, exist_ok=True)
        with open(args.records_out, "w") as f:
            json.dump(full, f, indent=1)
        records_file = args.records_out
    except OSError as e:
        print(f"bench.py: could not write {args.records_out}: {e}", file=sys.stderr)
    print(assemble_line(head, records, records_file), flush=True)
    return 0


def vendor_gemm_calibration(ms=(512, 2048, 4096), shapes=((14336, 4096), (4096, 14336)), reps=20):
    """torch.matmul in fp16 (fp32 accumulate inside the vendor library) at the prefill shapes, timed with events on
    torch's stream after a warm-up, rotating over enough weight copies to stay out of the last-level cache.  Not
    part of the product path: a yardstick for what fp16 MFMA sustains on this device under a dense matmul."""
    import torch
    out = {}
    dev = torch.device("cuda:0")
    for n, k in shapes:
        copies = 6
        ws = [torch.randn(n, k, device=dev, dtype=torch.float16) * 0.02 for _ in range(copies)]
        for m in ms:
            x = torch.randn(m, k, device=dev, dtype=torch.float16)
            for w in ws:
                torch.matmul(x, w.t())
            torch.cuda.synchronize()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            for _ in range(reps):
                for w in ws:
                    torch.matmul(x, w.t())
            e1.record()
            torch.cuda.synchronize()
            us = e0.elapsed_time(e1) * 1e3 / (reps * copies)
            tf = 2.0 * m * n * k / us / 1e6
            out[f"{k}x{n}.m{m}"] = {"us": round(us, 2), "TFLOPs": round(tf, 1), "frac_of_mfma_peak": round(tf / 2500.0, 4)}
    return out


if __name__ == "__main__":
    sys.exit(main())
