"""Throughput records of the quantized GGUF path, one per op and configuration, in the shape of the
reference's `KernelThroughputRecord`
(/root/reference/packages/tassadar-executor/src/kernel-optimization-parity.ts:26-59: targetModel,
device, hardwareRef, opRef, kernelRef, graphDigest, tokensPerSecond), plus the `/health`-shaped
object a Psionic server reports (/root/reference/apps/pylon/packages/runtime/src/cli.ts:1181 reads
`execution_engine` / `backend`, :1206-1213 `default_model` / `model` / `models`).

    python -m openagents_amd.records [--out DIR] [--configs 1,3,4,5] [--samples 9]

writes one JSON file per record and `health.json` into DIR and prints a one-line summary per record.
`bench.py` calls the same functions for the records it carries beside its headline.

Every figure is measured on graph replays (the launches of one sample are one HIP graph), with HIP
events on the launch stream; weights rotate over enough distinct device copies to defeat the 256 MB
last-level cache where the op is memory-bound.  `graphDigest` is the SHA-256 of the record's shape
tag and of the exact weight bytes the kernel read, so a record can be bound to the artifact a
validator replays.  `not_measured` lists what the record deliberately leaves out.
"""
from __future__ import annotations

import argparse
import hashlib
import json
import os
import sys
import time

import numpy as np

from . import _ffi, quantize
from ._ffi import ACT_Q8, Q4_0, Q4_K, Q6_K, Q8_0
from .backend import HipBackend, act_type_for, matvec_plan, prefill_plan, row_bytes

HBM_PEAK_GBS = 8000.0
MFMA_F16_PEAK_TFLOPS = 2500.0
TARGET_MODEL = "llama-3-8b-shaped-synthetic"
DEVICE_CLASS = "hip"
FMT_NAME = {Q4_0: "q4_0", Q8_0: "q8_0", Q4_K: "q4_K", _ffi.Q5_K: "q5_K", Q6_K: "q6_K"}


def hardware_ref(be: HipBackend) -> str:
    return f"amd-instinct-mi355x-{be.arch.split(':')[0]}-{be.compute_units}cu"


def graph_digest(tag: str, *blocks: np.ndarray) -> str:
    h = hashlib.sha256(tag.encode())
    for b in blocks:
        h.update(np.ascontiguousarray(b).view(np.uint8).reshape(-1).data)
    return h.hexdigest()


def stats(samples_us) -> dict:
    a = np.sort(np.asarray(samples_us, dtype=np.float64))
    return {"median_us": round(float(np.median(a)), 3), "p10_us": round(float(np.quantile(a, 0.1)), 3),
            "p90_us": round(float(np.quantile(a, 0.9)), 3), "samples": int(a.size)}


def time_graph(be: HipBackend, graph, launches_per_replay: int, samples: int = 9, replays: int = 3, warmup: int = 2):
    """Per-launch microseconds of `samples` timed groups of `replays` graph replays each."""
    for _ in range(warmup):
        be.launch_graph(graph)
    be.sync()
    ev = [be.event() for _ in range(samples + 1)]
    be.record(ev[0])
    for i in range(samples):
        for _ in range(replays):
            be.launch_graph(graph)
        be.record(ev[i + 1])
    be.sync()
    out = [be.elapsed_us(ev[i], ev[i + 1]) / (replays * launches_per_replay) for i in range(samples)]
    for e in ev:
        be.destroy_event(e)
    return out


def record(be: HipBackend, op_ref: str, kernel_ref: str, digest: str, tokens_per_second: float, **extra) -> dict:
    rec = {"targetModel": TARGET_MODEL, "device": DEVICE_CLASS, "hardwareRef": hardware_ref(be), "opRef": op_ref,
           "kernelRef": kernel_ref, "graphDigest": digest, "tokensPerSecond": round(float(tokens_per_second), 2)}
    rec.update(extra)
    return rec


def seeded_weights(seed: int, n: int, k: int) -> np.ndarray:
    return np.random.default_rng(seed).standard_normal((n, k), dtype=np.float32) * np.float32(0.02)


def matvec_kernel_name(qtype: int, ns, k: int, batch: int, cus: int, x_is_f32: bool = True) -> str:
    p = matvec_plan(qtype, ACT_Q8, sum(ns), k, batch, cus, x_is_f32)
    f = FMT_NAME[qtype]
    if p.mfma:
        return f"psn_quantize_q8_K + psn_mvm_{f}_q8_" + ("t8" if (k // 256) // p.mfma > 4 else "p4")
    if p.stream:
        return f"psn_mvs_{f}_q8_g{p.lanes_per_row}" + {1: "_lds", 2: "_xf"}[p.stage_lds] + f"_s{len(ns)}"
    return f"psn_mv_{f}_q8_g{p.lanes_per_row}_r{p.rows_in_flight}_b{p.batch_tile}" + {0: "", 1: "_lds", 2: "_xf"}[p.stage_lds]


def copies_for(nbytes: int, floor: int = 2) -> int:
    """Distinct device copies so that a rotation walks through more than 600 MB."""
    return max(floor, int(600e6 // nbytes) + 1)


def upload_copies(be: HipBackend, qtype: int, blocks: np.ndarray, n: int, k: int) -> list:
    return [be.upload_weight(qtype, blocks, n, k) for _ in range(copies_for(blocks.nbytes))]


def matvec_record(be: HipBackend, ws: list, blocks: np.ndarray, batch: int, op_ref: str, samples: int, seed: int) -> dict:
    """One matrix (device copies `ws` of the host `blocks`), fp32 activations in, activation scheme Q8,
    fp32 out, `batch` columns."""
    qtype, n, k, copies = ws[0].qtype, ws[0].n, ws[0].k, len(ws)
    x = be.upload(np.random.default_rng(seed).standard_normal((batch, k), dtype=np.float32))
    y = be.alloc(batch * n * 4)
    be.reserve(k, batch)
    be.begin_capture()
    for w in ws:
        be.quantized_matvec(w, x, y, batch, ACT_Q8)
    g = be.end_capture()
    st = stats(time_graph(be, g, copies, samples))
    be.destroy_graph(g)
    extra = {}
    if batch > 1:
        # the same projection fed with activations that are already quantized (what a fused producer hands over)
        xq = be.quantize_activations(x, k, batch, act_type_for(qtype))
        be.begin_capture()
        for w in ws:
            be.quantized_matvec_q8(w, xq, y, batch)
        g = be.end_capture()
        extra["timing_prequantized_input"] = stats(time_graph(be, g, copies, samples))
        be.destroy_graph(g)
    nbytes = n * row_bytes(qtype, k) + batch * 4 * (n + k)
    gbs = nbytes / st["median_us"] / 1e3
    return record(be, op_ref, matvec_kernel_name(qtype, [n], k, batch, be.compute_units),
                  graph_digest(f"{op_ref}:{FMT_NAME[qtype]}:n{n}:k{k}:b{batch}", blocks),
                  batch * 1e6 / st["median_us"], shape={"N": n, "K": k, "batch": batch, "format": FMT_NAME[qtype]},
                  timing=st, algorithmic_bytes=int(nbytes), GBps=round(gbs, 1), bound="hbm",
                  frac_of_roofline=round(gbs / HBM_PEAK_GBS, 4), weight_copies=copies, **extra,
                  tokens_definition="activation columns through this one projection per second",
                  not_measured=["end-to-end model tokens/s (this record is one projection)", "host-side launch cost (graph replay)"])


def config1(be: HipBackend, samples: int = 9, seed: int = 11, cpu: bool = True) -> list:
    """Q8_0 4096x4096, batch 1: the reference's own CPU-runnable case, timed here on the GPU and (cpu=True)
    on the host cores through the CPU oracle."""
    n = k = 4096
    w = seeded_weights(seed, n, k)
    blocks = quantize.quantize_q8_0(w)
    ws = upload_copies(be, Q8_0, blocks, n, k)
    rec = matvec_record(be, ws, blocks, 1, "matvec.q8_0.4096x4096.b1", samples, seed + 1)
    for w in ws:
        w.buf.free()
    if cpu:
        import oracle
        x = np.random.default_rng(seed + 1).standard_normal(k, dtype=np.float32)
        nbytes = rec["algorithmic_bytes"]
        cpu_rec = {}
        for label, threads in (("threads_1", 1), ("threads_all", oracle.max_threads())):
            reps, t0 = 0, time.perf_counter()
            while time.perf_counter() - t0 < 1.0:
                oracle.matvec(oracle.Q8_0, oracle.ACT_Q8, blocks, x, n, k, nthreads=threads)
                reps += 1
            dt = (time.perf_counter() - t0) / reps
            cpu_rec[label] = {"threads": threads, "us": round(dt * 1e6, 1), "GBps": round(nbytes / dt / 1e9, 2)}
        rec["cpu_reference_path"] = cpu_rec
    return [rec]


def config3(be: HipBackend, samples: int = 9, seed: int = 31, weights=None) -> list:
    """Q4_K 4096->14336 and 14336->4096 at batch 1, 2, 4, 8.  `weights` = {(n, k): blocks} reuses matrices."""
    out = []
    for n, k in ((14336, 4096), (4096, 14336)):
        blocks = weights[(n, k)] if weights and (n, k) in weights else quantize.quantize_q4_K(seeded_weights(seed + n % 7, n, k))
        ws = upload_copies(be, Q4_K, blocks, n, k)
        for batch in (1, 2, 4, 8):
            out.append(matvec_record(be, ws, blocks, batch, f"matvec.q4_K.{k}x{n}.b{batch}", samples, seed + batch))
        for w in ws:
            w.buf.free()
    return out


def prefill_kernel_name(fmt: str, m: int, n: int, k: int, cus: int, qtype: int | None = None):
    tm, tn, sp, wv = prefill_plan(m, n, k, cus, qtype)
    name = {64: f"psn_prefill_{fmt}_skinny", 32: f"psn_prefill_{fmt}_wide", 128: f"psn_prefill_{fmt}_unpack + psn_prefill_dense_f16" + ("_m128" if tm == 128 else "")}.get(wv, f"psn_prefill_{fmt}_m{tm}_n{tn}" + {4: "", 16: "_ws"}.get(wv, ""))
    return name, sp


def config4(be: HipBackend, samples: int = 7, seed: int = 41, weights=None, ms=(64, 512, 2048)) -> list:
    """Quantized prefill matmul, Q4_0 and Q8_0, both shapes, M = 64 / 512 / 2048: twelve cells."""
    out = []
    for qtype, quant in ((Q4_0, quantize.quantize_q4_0), (Q8_0, quantize.quantize_q8_0)):
        fmt = FMT_NAME[qtype]
        for n, k in ((14336, 4096), (4096, 14336)):
            blocks = weights[(qtype, n, k)] if weights and (qtype, n, k) in weights else quant(seeded_weights(seed + n % 7, n, k))
            ws = upload_copies(be, qtype, blocks, n, k)
            copies = len(ws)
            digest = graph_digest(f"prefill:{fmt}:n{n}:k{k}", blocks)
            for m in ms:
                x = be.upload(np.random.default_rng(seed + m).standard_normal((m, k), dtype=np.float32).astype(np.float16))
                y = be.alloc(m * n * 4)
                be.begin_capture()
                for w in ws:
                    be.quantized_matmul(w, x, y, m)
                g = be.end_capture()
                st = stats(time_graph(be, g, copies, samples, replays=2 if m >= 512 else 3))
                be.destroy_graph(g)
                flops = 2.0 * m * n * k
                nbytes = n * row_bytes(qtype, k) + m * k * 2 + m * n * 4
                t_us = st["median_us"]
                bound_us = max(flops / (MFMA_F16_PEAK_TFLOPS * 1e6), nbytes / (HBM_PEAK_GBS * 1e3))
                bound = "mfma" if flops / (MFMA_F16_PEAK_TFLOPS * 1e6) >= nbytes / (HBM_PEAK_GBS * 1e3) else "hbm"
                kname, sp = prefill_kernel_name(fmt, m, n, k, be.compute_units, qtype)
                packed_extra = {}
                if m >= 2048:
                    # the same projection with the dequantization hoisted out of the call (psn_prefill_pack once, then
                    # psn_qmatmul_prefill_packed): three packed copies rotate (2 bytes per weight each)
                    packs = [be.pack_for_prefill(w) for w in ws[:3]]
                    be.begin_capture()
                    for pk in packs:
                        be.quantized_matmul_packed(pk, x, y, m, n, k)
                    gp = be.end_capture()
                    sp_ = stats(time_graph(be, gp, len(packs), samples, replays=2))
                    be.destroy_graph(gp)
                    for pk in packs:
                        pk.free()
                    packed_extra = {"timing_packed_weights": {**sp_, "TFLOPs": round(flops / sp_["median_us"] / 1e6, 1),
                                                              "frac_of_mfma_peak": round(flops / sp_["median_us"] / 1e6 / MFMA_F16_PEAK_TFLOPS, 4),
                                                              "kernelRef": "psn_prefill_dense_f16 or psn_prefill_dense_f16_m128 (by shape)",
                                                              "note": "weights dequantized to fp16 fragments once beforehand (psn_prefill_pack, 2 bytes per weight resident)"}}
                out.append(record(be, f"prefill.{fmt}.{k}x{n}.m{m}", kname, digest, m * 1e6 / t_us,
                                  shape={"M": m, "N": n, "K": k, "format": fmt, "ksplit": sp}, timing=st,
                                  TFLOPs=round(flops / t_us / 1e6, 1), GBps=round(nbytes / t_us / 1e3, 1),
                                  algorithmic_bytes=int(nbytes), flops=int(flops), bound=bound,
                                  roofline_us=round(bound_us, 2), frac_of_roofline=round(bound_us / t_us, 4),
                                  frac_of_mfma_peak=round(flops / t_us / 1e6 / MFMA_F16_PEAK_TFLOPS, 4), weight_copies=copies,
                                  tokens_definition="prompt rows through this one projection per second",
                                  not_measured=["end-to-end prefill tokens/s (this record is one projection)",
                                                "host-side launch cost (graph replay)"], **packed_extra))
                x.free()
                y.free()
            for w in ws:
                w.buf.free()
    return out


def config5(be: HipBackend, samples: int = 7, seed: int = 0, ctx: int = 2048, layers: int = 32) -> list:
    """The synthetic Llama-3-8B-shaped Q4_K decode step at batch 1, context `ctx`, Q6_K LM head."""
    from .decode import DecodeStep, LlamaShape, synthetic_weights
    shape = LlamaShape(n_layers=layers)
    t0 = time.time()
    protos = {}
    weights = synthetic_weights(be, shape, seed, keep_host=protos)
    step = DecodeStep(be, shape, weights, ctx)
    rng = np.random.default_rng(seed + 1)
    pos = ctx - 1
    kv = rng.standard_normal((pos, shape.kv_dim), dtype=np.float32).astype(np.float16)
    for li in range(shape.n_layers):
        step.k_cache[li].upload(kv)
        step.v_cache[li].upload(kv)
    x0 = rng.standard_normal(shape.hidden, dtype=np.float32)
    step.x.upload(x0)
    setup_s = time.time() - t0
    full, mv = step.capture(pos), step.capture(pos, matvecs_only=True)
    st_full = stats(time_graph(be, full, 1, samples, replays=3))
    st_mv = stats(time_graph(be, mv, 1, samples, replays=3))
    step.x.upload(x0)
    be.launch_graph(full)
    logits = step.logits.download(np.float32, (shape.vocab,))
    be.destroy_graph(full)
    be.destroy_graph(mv)
    mbytes = step.matvec_bytes()
    t_full, t_mv = st_full["median_us"], st_mv["median_us"]
    digest = graph_digest(f"decode-step:l{layers}:ctx{ctx}:h{shape.hidden}:ffn{shape.ffn}:v{shape.vocab}",
                          *[protos[name] for name in sorted(protos)])
    launches = step.launches_per_token
    rec = record(be, "decode.step.q4_K.b1", f"psn decode-step graph ({launches} launches: psn_mvs_q4_K_q8_g*_xn_s*, psn_mvs_q4_K_q8_g*_lds_s1, "
                 "psn_mvs_q6_K_q8_g16_xn_s1, psn_attn_partial_rope, psn_attn_combine, psn_swiglu, psn_rope_table)",
                 digest, 1e6 / t_full, shape={"layers": layers, "hidden": shape.hidden, "heads": shape.n_heads, "kv_heads": shape.n_kv_heads,
                                              "head_dim": shape.head_dim, "ffn": shape.ffn, "vocab": shape.vocab, "context": ctx,
                                              "weights": "Q4_K projections, Q6_K LM head"},
                 timing=st_full, ms_per_token=round(t_full / 1e3, 4), matvec_ms=round(t_mv / 1e3, 4), glue_ms=round((t_full - t_mv) / 1e3, 4),
                 matvec_share=round(t_mv / t_full, 4), matvec_GBps=round(mbytes / t_mv / 1e3, 1), matvec_bytes_per_token=int(mbytes),
                 bound="hbm", frac_of_roofline=round(mbytes / t_mv / 1e3 / HBM_PEAK_GBS, 4), launches_per_token=launches,
                 logits_finite=bool(np.all(np.isfinite(logits))), setup_s=round(setup_s, 1),
                 data="random-init weights (one unique layer copied to every layer's own allocation), fp16 N(0,1) KV cache",
                 tokens_definition="decoded tokens per second at batch 1 (whole step, graph replay)",
                 not_measured=["sampling", "tokenizer", "host loop", "prompt prefill"])
    return [rec]


def read_calibration(be: HipBackend, samples: int = 7) -> dict:
    """What a kernel that only reads (no decode, one partial sum per thread) reaches on this device at the
    byte counts of the four Llama-3-8B launches: the ceiling the streaming matvecs are compared with."""
    out = {}
    for name, nbytes in (("o_9.4MB", 9_437_184), ("qkv_14.2MB", 14_155_776), ("down_33MB", 33_030_144), ("gate_up_66MB", 66_060_288)):
        copies = copies_for(nbytes)
        srcs = [be.alloc(nbytes) for _ in range(copies)]
        for s in srcs:
            s.fill_zero()
        sink = be.alloc(1 << 20)
        be.begin_capture()
        for s in srcs:
            be.calibrate_read(s, nbytes, be.compute_units, 512, 0, sink)
        g = be.end_capture()
        st = stats(time_graph(be, g, copies, samples))
        be.destroy_graph(g)
        for s in srcs:
            s.free()
        out[name] = {"bytes": nbytes, **st, "GBps": round(nbytes / st["median_us"] / 1e3, 1)}
    return out


def health(be: HipBackend, models=(TARGET_MODEL,)) -> dict:
    """What a Psionic server would answer on /health with this backend behind it."""
    return {"status": "ok", "execution_engine": "psionic", "backend": "hip", "default_model": models[0], "model": models[0],
            "models": list(models), "device": hardware_ref(be), "abi_version": int(_ffi.load().psn_abi_version())}


def main(argv=None):
    ap = argparse.ArgumentParser()
    ap.add_argument("--out", default="psn_records")
    ap.add_argument("--configs", default="1,3,4,5")
    ap.add_argument("--samples", type=int, default=9)
    ap.add_argument("--no-cpu", action="store_true")
    args = ap.parse_args(argv)
    os.makedirs(args.out, exist_ok=True)
    be = HipBackend(0)
    be.reserve_prefill(14336, 4096)      # the dense prefill family's workspace, before any graph refers to the stream's workspace
    recs = []
    todo = set(args.configs.split(","))
    if "1" in todo:
        recs += config1(be, args.samples, cpu=not args.no_cpu)
    if "3" in todo:
        recs += config3(be, args.samples)
    if "4" in todo:
        recs += config4(be, args.samples)
    if "5" in todo:
        recs += config5(be, args.samples)
    for r in recs:
        with open(os.path.join(args.out, r["opRef"] + ".json"), "w") as f:
            json.dump(r, f, indent=1)
        print(f"{r['opRef']:40s} {r['kernelRef'][:48]:48s} {r['timing']['median_us']:10.2f} us  frac {r['frac_of_roofline']:.3f}", flush=True)
    with open(os.path.join(args.out, "health.json"), "w") as f:
        json.dump(health(be), f, indent=1)
    return 0


if __name__ == "__main__":
    sys.exit(main())
