"""The committed fixtures (tests/golden/psn_golden.npz, written by tests/golden/make_fixtures.py) against the
oracle as built now (CPU) and against the HIP kernels through the C ABI (-m gpu).  Quantized bytes and the
integer-path results must match bit for bit; fp32 accumulations may differ in the last bits between builds
of the oracle (OpenMP thread count, compiler) and between CPU and GPU, so they are held to 2e-6 / 2e-5 of
the output scale (the gate of the path is 1e-3)."""
import os

import numpy as np
import pytest

import ggufref as G

GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "psn_golden.npz")
N, K = 8, 512
FORMATS = {"q4_0": 2, "q8_0": 8, "q4_K": 12, "q6_K": 14, "q5_K": 13}


@pytest.fixture(scope="module")
def gold():
    with np.load(GOLD, allow_pickle=False) as z:
        return {k: z[k] for k in z.files}


@pytest.mark.parametrize("name", list(FORMATS))
def test_oracle_reproduces_golden_blocks_and_outputs(orc, gold, name):
    t = FORMATS[name]
    blocks = orc.quantize(t, gold[f"{name}_w"])
    assert np.array_equal(blocks, gold[f"{name}_blocks"])
    assert np.array_equal(orc.dequantize(t, blocks, K), gold[f"{name}_deq"])
    x = gold[f"{name}_x"]
    assert np.array_equal(orc.matvec(t, orc.ACT_Q8, blocks, x, N, K, nthreads=1), gold[f"{name}_y_q8"])
    assert G.max_rel_err(orc.matvec(t, orc.ACT_F32, blocks, x, N, K), gold[f"{name}_y_f32"]) < 2e-6
    if f"{name}_xh" in gold:
        assert G.max_rel_err(orc.prefill(t, blocks, gold[f"{name}_xh"], N, K), gold[f"{name}_y_prefill"]) < 2e-6


@pytest.mark.parametrize("name", ["q4_K", "q5_K"])
def test_oracle_reproduces_golden_batch8_outputs(orc, gold, name):
    t = FORMATS[name]
    blocks, x = gold[f"batch8_{name}_blocks"], gold[f"batch8_{name}_x"]
    assert np.array_equal(orc.matvec(t, orc.ACT_Q8, blocks, x, 32, K, nthreads=1), gold[f"batch8_{name}_y_q8"])


def test_oracle_reproduces_golden_activation_blocks(orc, gold):
    assert np.array_equal(orc.quantize(orc.Q8_0, gold["act_x"]), gold["act_q8_0"])
    assert np.array_equal(orc.quantize(orc.Q8_K, gold["act_x"]), gold["act_q8_K"])


def test_golden_blocks_parse_to_their_dequantized_values(gold):
    """The fixture is self-consistent under the independent element-index parsers (no oracle involved)."""
    d, q = G.parse_q4_0(gold["q4_0_blocks"], K)
    assert np.array_equal((d[:, :, None] * q).reshape(N, K).astype(np.float32), gold["q4_0_deq"])
    d, q = G.parse_q8_0(gold["q8_0_blocks"], K)
    assert np.array_equal((d[:, :, None] * q).reshape(N, K).astype(np.float32), gold["q8_0_deq"])
    d, dmin, sc, mn, q = G.parse_q4_K(gold["q4_K_blocks"], K)
    f = np.float32
    ref = (d.astype(f)[:, :, None] * sc.astype(f)).repeat(32, axis=2) * q.astype(f) - (dmin.astype(f)[:, :, None] * mn.astype(f)).repeat(32, axis=2)
    assert np.array_equal(ref.reshape(N, K), gold["q4_K_deq"])
    d, scales, q = G.parse_q6_K(gold["q6_K_blocks"], K)
    ref = (d.astype(f)[:, :, None] * scales.astype(f)).repeat(16, axis=2) * q.astype(f)
    assert np.array_equal(ref.reshape(N, K), gold["q6_K_deq"])


@pytest.mark.gpu
@pytest.mark.parametrize("name", list(FORMATS))
def test_gpu_matches_golden(hip, gold, name):
    from openagents_amd import _ffi
    t = FORMATS[name]
    blocks, x = gold[f"{name}_blocks"], gold[f"{name}_x"]
    y = hip.matvec_host(t, blocks, x, N, K, _ffi.ACT_Q8)
    assert G.max_rel_err(y, gold[f"{name}_y_q8"]) < 2e-5
    y = hip.matvec_host(t, blocks, x, N, K, _ffi.ACT_F32)
    assert G.max_rel_err(y, gold[f"{name}_y_f32"]) < 2e-5
    if f"{name}_xh" in gold:
        y = hip.matmul_host(t, blocks, gold[f"{name}_xh"], N, K)
        assert G.max_rel_err(y, gold[f"{name}_y_prefill"]) < 2e-5


@pytest.mark.gpu
@pytest.mark.parametrize("name", ["q4_K", "q5_K"])
def test_gpu_small_batch_kernels_match_golden(hip, gold, name):
    """Batch 8 and batch 4 of a 32-row matrix: the default plan puts these on the int8-MFMA kernels."""
    from openagents_amd import _ffi, backend
    t = FORMATS[name]
    blocks, x, want = gold[f"batch8_{name}_blocks"], gold[f"batch8_{name}_x"], gold[f"batch8_{name}_y_q8"]
    assert backend.matvec_plan(t, _ffi.ACT_Q8, 32, K, 8, hip.compute_units, True).mfma > 0
    for b in (8, 4):
        y = hip.matvec_host(t, blocks, x[:b], 32, K, _ffi.ACT_Q8)
        assert G.max_rel_err(y, want[:b]) < 2e-5


@pytest.mark.gpu
def test_gpu_activation_quantizers_match_golden_bytes(hip, gold):
    from openagents_amd import _ffi
    from openagents_amd.backend import actq_layout
    x = gold["act_x"]
    b = x.shape[0]
    xb = hip.upload(x)
    for act, key in ((_ffi.Q8_0, "act_q8_0"), (_ffi.Q8_K, "act_q8_K")):
        info = actq_layout(act, K, b)
        raw = hip.quantize_activations(xb, K, b, act).download(np.uint8, (int(info.bytes),))
        qs = raw[:b * K].view(np.int8).reshape(b, K)
        if act == _ffi.Q8_0:
            blk = gold[key].reshape(b, K // 32, 34)
            assert np.array_equal(qs.reshape(b, K // 32, 32), blk[:, :, 2:].view(np.int8))
            d = raw[info.off_d:info.off_d + b * (K // 32) * 4].view(np.float32).reshape(b, K // 32)
            assert np.array_equal(d.astype(np.float16).view(np.uint16), blk[:, :, :2].copy().view(np.uint16).reshape(b, K // 32))
        else:
            blk = gold[key].reshape(b, K // 256, 292)
            assert np.array_equal(qs.reshape(b, K // 256, 256), blk[:, :, 4:260].view(np.int8))
            d = raw[info.off_d:info.off_d + b * (K // 256) * 4].view(np.float32).reshape(b, K // 256)
            assert np.array_equal(d, blk[:, :, :4].copy().view(np.float32).reshape(b, K // 256))
            bs = raw[info.off_s:info.off_s + b * (K // 16) * 2].view(np.int16).reshape(b, K // 256, 16)
            assert np.array_equal(bs, blk[:, :, 260:].copy().view(np.int16).reshape(b, K // 256, 16))
