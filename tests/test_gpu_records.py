"""The throughput records as the reference's acceptance rule wants them
(/root/reference/packages/tassadar-executor/src/kernel-optimization-parity.ts:26-59 for the record, :118-136 for
"parity before throughput, both bound to one graphDigest"): built on the device with few samples and a checker on
the CPU oracle, every record must carry the reference's keys, a roofline object with 0 < fraction <= 1, a parity
verdict that passes, a digest that is stable across runs, and a kernelRef naming kernels the module really holds."""
import json

import numpy as np
import pytest

import bench
from openagents_amd import _ffi
from openagents_amd import records as R

pytestmark = pytest.mark.gpu

REFERENCE_KEYS = {"targetModel", "device", "hardwareRef", "opRef", "kernelRef", "graphDigest", "tokensPerSecond"}


def kernels_of(rec):
    ref = rec["kernelRef"]
    if "(" in ref:                                            # the decode-step record: "psn decode-step graph (N launches: a, b, c)"
        ref = ref[ref.index(":") + 1:ref.rindex(")")].replace(",", " + ")
    return [k.strip() for k in ref.split("+") if k.strip()]


def check(hip, rec):
    assert set(rec) >= REFERENCE_KEYS | {"roofline", "parity", "not_measured", "timing"}, rec["opRef"]
    assert rec["device"] == "hip" and rec["tokensPerSecond"] > 0 and len(rec["graphDigest"]) == 64
    assert 0 < rec["roofline"]["fraction"] <= 1 and rec["roofline"]["bound"] in ("hbm", "mfma"), (rec["opRef"], rec["roofline"])
    assert rec["parity"]["status"] == "pass" and rec["parity"]["value"] < rec["parity"]["gate"] == 1e-3, (rec["opRef"], rec["parity"])
    names = kernels_of(rec)
    assert names, rec["kernelRef"]
    for k in names:
        assert hip.lib.psn_module_has_kernel(hip.module, k.encode()) == 0, (rec["opRef"], k)
    json.dumps(rec)


def test_matvec_and_prefill_records(hip, orc):
    checker = bench.OracleChecker()
    hip.reserve_prefill(14336, 4096)
    recs = R.config1(hip, 2, checker=checker, cpu_path=None)
    recs += R.config4(hip, 2, ms=(64, 512), checker=checker, shapes=((14336, 4096),), formats=(_ffi.Q4_0,))
    assert [r["opRef"] for r in recs] == ["matvec.q8_0.4096x4096.b1", "prefill.q4_0.4096x14336.m64", "prefill.q4_0.4096x14336.m512"]
    for r in recs:
        print(f"record {r['opRef']}: {r['kernelRef']} frac={r['roofline']['fraction']} parity={r['parity']['value']:.2e}", flush=True)
        check(hip, r)
    assert recs[0]["kernelRef"].startswith("psn_mvs_q8_0") and recs[1]["roofline"]["bound"] == "hbm" and recs[2]["roofline"]["bound"] == "mfma"
    again = R.config1(hip, 2, checker=None)
    assert again[0]["graphDigest"] == recs[0]["graphDigest"]                       # same seeded bytes, same digest
    assert again[0]["parity"]["status"] == "not_checked" and any("parity" in t for t in again[0]["not_measured"])
    assert again[0]["kernelRef"] == recs[0]["kernelRef"]


def test_small_batch_record_names_both_launches(hip, orc):
    """Q4_K at batch 8 on fp32 input runs a quantize launch and the int8-MFMA kernel: both must be in kernelRef."""
    checker = bench.OracleChecker()
    from openagents_amd import quantize
    n, k = 2048, 4096
    blocks = quantize.quantize_q4_K(R.seeded_weights(77, n, k))
    ws = [hip.upload_weight(_ffi.Q4_K, blocks, n, k) for _ in range(3)]
    rec = R.matvec_record(hip, ws, blocks, 8, "matvec.q4_K.4096x2048.b8", 2, 78, checker)
    print(f"record {rec['opRef']}: {rec['kernelRef']}", flush=True)
    check(hip, rec)
    assert len(kernels_of(rec)) == 2 and "timing_prequantized_input" in rec


def test_decode_step_record_and_worker_attachment(hip, orc):
    checker = bench.OracleChecker()
    rec, head = R.config5(hip, 2, ctx=256, layers=2, checker=checker)
    print(f"record {rec['opRef']}: {rec['kernelRef']} parity={rec['parity']['value']:.2e}", flush=True)
    check(hip, rec)
    print(f"record {head['opRef']}: {head['kernelRef']} parity={head['parity']['value']:.2e}", flush=True)
    check(hip, head)                                         # the Q6_K LM head on its own
    assert head["opRef"].startswith("matvec.q6_K.4096x128256") and "q6_K" in head["kernelRef"]
    assert rec["launches_per_token"] == 2 * 6 + 2 and "xnp" in rec["kernelRef"] and 0 < rec["matvec_share"] <= 1   # SwiGLU inside gate|up
    assert any(k.startswith("psn_attn") for k in kernels_of(rec)) and any("q6_K" in k for k in kernels_of(rec))
    att = R.worker_attachment([rec], updated_at_ms=5)
    assert att["workers"][0]["ready"] is True and att["workers"][0]["evidence_digest"] == R.record_digest(rec)
    h = R.health(hip)
    assert h["execution_engine"] == "psionic" and h["backend"] == "hip" and h["models"] == [h["default_model"]]


def test_wide_model_shape_against_the_cpu_path(hip, orc):
    """A 70B-class layer shape (hidden 8192, 64 query / 8 kv heads, FFN 28672): the norm-fused projections stage
    8192 values with eight-wave workgroups, the SwiGLU pair kernel runs at K = 8192, the down projection's rows
    (112 chunks) are too long for the streaming kernels, the attention group is eight heads.  Two layers from a
    512-token cache; the last layer's launches are recomputed on the CPU from the device's own inputs."""
    from openagents_amd.decode import DecodeStep, LlamaShape, synthetic_weights
    shape = LlamaShape(hidden=8192, n_heads=64, n_kv_heads=8, ffn=28672, vocab=4096, n_layers=2)
    protos = {}
    weights = synthetic_weights(hip, shape, 3, head_rows_unique=4096, keep_host=protos)
    ctx = 512
    step = DecodeStep(hip, shape, weights, ctx)
    assert step.fused_norm and step.fused_swiglu == [True, True]
    rng = np.random.default_rng(4)
    pos = ctx - 1
    kv = rng.standard_normal((pos, shape.kv_dim), dtype=np.float32).astype(np.float16)
    for li in range(shape.n_layers):
        step.k_cache[li].upload(kv)
        step.v_cache[li].upload(kv)
    step.x.upload(rng.standard_normal(shape.hidden, dtype=np.float32))
    print("wide shape: enqueue", flush=True)
    step.enqueue(pos)
    hip.sync()
    got = {"x": step.x.download(np.float32, (shape.hidden,)), "down": step.down.download(np.float32, (shape.hidden,)),
           "act": step.act.download(np.float32, (shape.ffn,)), "logits": step.logits.download(np.float32, (shape.vocab,))}
    assert all(np.all(np.isfinite(v)) for v in got.values())
    ref = bench.OracleChecker().decode_last_layer(shape, protos, got)
    for name in ("act", "down", "logits"):
        verdict = R.parity_of(got[name], ref[name], "Q8", name)
        print(f"wide shape {name}: {verdict['value']:.2e}", flush=True)
        assert verdict["status"] == "pass", (name, verdict)
