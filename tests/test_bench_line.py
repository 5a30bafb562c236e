"""The last line bench.py prints must stay a single JSON object of fewer than 2000 characters carrying the
headline, `roofline`, `cpu_baseline`, the parity verdict and a compact summary of the other configurations,
whatever the records hold; and the record helpers must produce the reference's KernelThroughputRecord keys
(/root/reference/packages/tassadar-executor/src/kernel-optimization-parity.ts:26-59) plus `roofline` and
`parity`.  Canned inputs: no GPU."""
import json
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)

import bench  # noqa: E402
from openagents_amd import records as R  # noqa: E402


class FakeBackend:
    arch = "gfx950:sramecc+:xnack-"
    compute_units = 256


def canned_records():
    be = FakeBackend()
    recs = []
    ok = R.parity_of(np.array([1.0, 2.0]), np.array([1.0, 2.0000001]), "Q8", "all outputs")
    recs.append(R.record(be, "matvec.q8_0.4096x4096.b1", "psn_mvs_q8_0_q8_g16_xf_s1", "d" * 64, 1e5, R.roofline_of("hbm", 2630.0), ok, ["x"]))
    for shape in ("4096x14336", "14336x4096"):
        for b in (1, 2, 4, 8):
            recs.append(R.record(be, f"matvec.q4_K.{shape}.b{b}", "psn_quantize_q8_K + psn_mvm_q4_K_q8_t8", "e" * 64, 1e5, R.roofline_of("hbm", 2900.0), ok))
    for fmt in ("q4_0", "q8_0"):
        for shape in ("4096x14336", "14336x4096"):
            for m, bound, a in ((64, "hbm", 1650.0), (512, "mfma", 677.0), (2048, "mfma", 985.0)):
                recs.append(R.record(be, f"prefill.{fmt}.{shape}.m{m}", f"psn_prefill_{fmt}_unpack + psn_prefill_dense_f16_m128", "f" * 64, 1e6,
                                     R.roofline_of(bound, a), None))
    recs.append(R.record(be, "decode.step.q4_K.b1", "psn decode-step graph (226 launches: " + ", ".join(f"psn_kernel_with_a_long_name_{i}" for i in range(12)) + ")",
                         "a" * 64, 602.27, R.roofline_of("hbm", 3929.2), ok, ["sampling"], matvec_share=0.6693))
    recs.append(R.record(be, "matvec.q6_K.4096x128256.b1", "psn_mvs_q6_K_q8_g16_xf_s1", "b" * 64, 1.2e4, R.roofline_of("hbm", 5400.0), ok))
    return recs


def canned_head():
    return {"value": 3518.3, "steps": 20, "warmup": 5, "ms_per_step": 1.1184, "launches_per_step": 128, "bytes_per_step": 3934781440,
            "roofline": {"bound": "hbm", "achieved": 4932.1, "peak": 8000.0, "unit": "GB/s", "frac": 0.6165, "traffic": 66512700,
                         "traffic_source": "x" * 200, "kernel": "psn_mvs_q4_0_q8_g16_xf_s2", "avg_launch_us": 13.421,
                         "algo_bytes_per_launch": 66191360, "launches_per_step": 32, "note": "n" * 300},
            "cpu_baseline": {"value": 24.91, "unit": "GB/s", "cores": 16, "kind": "port", "sample": "s" * 400,
                             "single_thread": {"value": 1.68, "unit": "GB/s", "cores": 1, "sample": "t" * 100},
                             "host": {"nproc": 256, "cpu_model": "AMD EPYC 9575F 64-Core Processor"}, "provenance": "p" * 200},
            "parity": {"value": 7.489e-07, "gate": 1e-3, "status": "pass"},
            "per_launch_us": {"qkv": 6.371, "o": 4.962, "gate_up": 13.901, "down": 10.652}, "two_streams_GBps": 4372.0}


def test_headline_line_is_short_and_complete():
    recs = canned_records()
    text = bench.assemble_line(canned_head(), recs, "gpurun_out/bench_records.json")
    assert "\n" not in text and len(text) < bench.MAX_LINE_CHARS, len(text)
    line = json.loads(text)
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling", "vs_baseline", "dtype",
                "data", "config", "roofline", "cpu_baseline", "parity", "configs"):
        assert key in line, key
    assert line["config"]["workload"].startswith("Q4_0 decode matvec") and "model" not in line["config"]
    assert set(line["roofline"]) >= {"bound", "achieved", "peak", "unit", "frac", "traffic"} and line["roofline"]["bound"] == "hbm"
    assert abs(line["roofline"]["frac"] - line["roofline"]["achieved"] / line["roofline"]["peak"]) < 1e-3
    assert set(line["cpu_baseline"]) >= {"value", "unit", "cores", "kind", "sample"} and line["cpu_baseline"]["kind"] == "port"
    assert line["vs_baseline"] is None and line["n_gpus"] == 1 and line["steps"] == 20 and line["warmup"] == 5
    c = line["configs"]
    assert c["c1_q8_0_4096"] == recs[0]["roofline"]["fraction"]
    assert [len(v) for v in c["c3_q4_K_b1248"].values()] == [4, 4]
    assert len(c["c4_m64_512_2048"]) == 4 and all(len(v) == 3 for v in c["c4_m64_512_2048"].values())
    assert c["c5"]["tok_s"] == 602.27 and c["c5"]["matvec_share"] == 0.6693 and c["c5"]["lm_head_q6_K_frac"] == 0.675
    assert c["parity_not_pass"] == 12                     # the twelve canned prefill records carry no verdict
    # without records (headline only) and without the CPU leg the line is still well formed
    head = canned_head()
    head["cpu_baseline"], head["parity"] = None, None
    line2 = json.loads(bench.assemble_line(head, None, None))
    assert line2["configs"] is None and line2["cpu_baseline"] is None and line2["roofline"]["kernel"]


def test_record_shape_matches_the_reference_record_plus_roofline_and_parity():
    recs = canned_records()
    for r in recs:
        # KernelThroughputRecord of the reference: these seven keys, device one of its classes
        assert set(r) >= {"targetModel", "device", "hardwareRef", "opRef", "kernelRef", "graphDigest", "tokensPerSecond"}
        assert r["device"] == "hip" and r["hardwareRef"] == "amd-instinct-mi355x-gfx950-256cu" and r["tokensPerSecond"] > 0
        assert set(r["roofline"]) == {"bound", "peak", "achieved", "fraction", "unit"} and 0 < r["roofline"]["fraction"] <= 1
        assert set(r["parity"]) >= {"status", "metric", "value", "gate"} and r["parity"]["status"] in ("pass", "fail", "not_checked")
        assert isinstance(r["not_measured"], list)
    unchecked = [r for r in recs if r["parity"]["status"] == "not_checked"]
    assert len(unchecked) == 12 and all(any("parity" in t for t in r["not_measured"]) for r in unchecked)
    bad = R.parity_of(np.array([1.0, 2.0]), np.array([1.0, 2.1]), "Q8", "x")
    assert bad["status"] == "fail" and bad["value"] > 1e-3
    nan = R.parity_of(np.array([1.0, np.nan]), np.array([1.0, 2.0]), "Q8", "x")
    assert nan["status"] == "fail"
    # the digest of a record is stable and changes with what was measured
    assert R.record_digest(recs[0]) == R.record_digest(dict(recs[0]))
    other = dict(recs[0], tokensPerSecond=recs[0]["tokensPerSecond"] + 1)
    assert R.record_digest(other) != R.record_digest(recs[0])
    assert R.graph_digest("t", np.arange(4, dtype=np.uint8)) != R.graph_digest("t", np.arange(1, 5, dtype=np.uint8))


def test_worker_attachment_has_the_reference_fields():
    """PsionicWorkerAttachment / PsionicWorkerRecord, /root/reference/crates/openagents-cloud-contract/src/lib.rs:1723-1745."""
    recs = canned_records()
    att = R.worker_attachment(recs, updated_at_ms=1234)
    assert set(att) == {"schema_version", "updated_at_ms", "workers"} and att["updated_at_ms"] == 1234
    (w,) = att["workers"]
    assert set(w) == {"product_id", "worker_id", "worker_kind", "ready", "crashed", "evidence_digest", "detail"}
    step = next(r for r in recs if r["opRef"].startswith("decode.step"))
    assert w["evidence_digest"] == R.record_digest(step) and w["crashed"] is False
    assert w["ready"] is False                               # twelve records carry no verdict: not ready
    passed = [r for r in recs if r["parity"]["status"] == "pass"]
    assert R.worker_attachment(passed)["workers"][0]["ready"] is True
    json.dumps(att)


def test_read_sweep_geometries_fit_a_compute_unit():
    geos = R.read_sweep_geometries(256)
    assert len(geos) >= 16 and len(set(geos)) == len(geos)
    for blocks, threads, depth in geos:
        per_cu = blocks // 256
        assert blocks % 256 == 0 and threads in (256, 512) and per_cu * threads <= 2048
        assert per_cu * (threads // 64) * depth * 1024 <= 160 * 1024


def test_measured_traffic_constants_are_the_ones_in_the_committed_profile():
    """bench.py's `roofline.traffic` figures are pasted from a rocprofv3 counter summary: every constant must
    still stand in that summary's table (a refreshed profile with an unrefreshed constant fails here), and the
    file must name the kernel of the headline's dominant launch."""
    text = open(os.path.join(ROOT, "profiles", "matvec_q4_0_llama3_8b_step.md")).read()
    assert bench.MEASURED_TRAFFIC_BYTES, "no traffic constants"
    for kernel, nbytes in bench.MEASURED_TRAFFIC_BYTES.items():
        assert f"{nbytes:,}".replace(",", " ") in text, (kernel, nbytes)
    assert "psn_mvs_q4_0_q8_g16_xf_s2" in text
