"""GGUF container: writer -> reader round trip (CPU) and file -> device -> matvec parity (GPU).

No .gguf file exists in the reference tree, so what is pinned here is the container layout as this
module states it (header fields, typed metadata, alignment, tensor table) and that quantized tensor
bytes reach the kernels unchanged; agreement with files written by other tools is not covered."""
import struct

import numpy as np
import pytest

import ggufref as G
from openagents_amd import gguf


def make_file(orc, path, alignment=32):
    k = 1024
    tensors, raw = [], {}
    for name, t, n in (("blk.0.attn_q.weight", orc.Q4_0, 48), ("blk.0.ffn_down.weight", orc.Q4_K, 40),
                       ("output.weight", orc.Q6_K, 72), ("blk.0.attn_k.weight", orc.Q8_0, 16), ("blk.0.ffn_up.weight", orc.Q5_K, 24)):
        blocks = orc.quantize(t, G.seeded_weights(1000 + n, n, k))
        raw[name] = (t, n, k, blocks)
        tensors.append((name, (k, n), t, blocks))
    norm = np.linspace(0.5, 1.5, 512, dtype=np.float32)
    tensors.append(("output_norm.weight", (512,), 0, norm.view(np.uint8)))
    md = {"general.architecture": (gguf.STRING, "llama"), "llama.block_count": (gguf.U32, 1),
          "llama.rope.freq_base": (gguf.F32, 500000.0), "general.file_type": (gguf.I32, -7),
          "tokenizer.ggml.tokens": (gguf.ARRAY, (gguf.STRING, ["<s>", "</s>", "héllo"])),
          "some.u64": (gguf.U64, 2 ** 40 + 3), "some.bool": (gguf.BOOL, True), "some.f64": (gguf.F64, 0.1),
          "some.i8s": (gguf.ARRAY, (gguf.I8, [-128, 0, 127]))}
    gguf.write_gguf(str(path), md, tensors, alignment)
    return raw, norm


@pytest.mark.parametrize("alignment", [32, 64, 4096])
def test_round_trip_header_metadata_and_tensor_bytes(orc, tmp_path, alignment):
    path = tmp_path / "m.gguf"
    raw, norm = make_file(orc, path, alignment)
    f = gguf.GGUFFile(str(path))
    assert f.version == 3 and f.alignment == alignment and f.data_start % alignment == 0
    assert f.metadata["general.architecture"] == "llama" and f.metadata["llama.block_count"] == 1
    assert f.metadata["llama.rope.freq_base"] == 500000.0 and f.metadata["general.file_type"] == -7
    assert f.metadata["tokenizer.ggml.tokens"] == ["<s>", "</s>", "héllo"]
    assert f.metadata["some.u64"] == 2 ** 40 + 3 and f.metadata["some.bool"] is True and f.metadata["some.i8s"] == [-128, 0, 127]
    assert list(f.tensors) == list(raw) + ["output_norm.weight"]
    for name, (t, n, k, blocks) in raw.items():
        info = f.tensors[name]
        assert (info.ggml_type, info.n, info.k, info.offset % alignment) == (t, n, k, 0)
        assert np.array_equal(f.data(name), blocks.reshape(-1))
    assert np.array_equal(f.data("output_norm.weight").view(np.float32), norm)
    # the first bytes are exactly the documented header
    head = open(path, "rb").read(24)
    assert head[:4] == b"GGUF" and struct.unpack("<IQQ", head[4:]) == (3, 6, 9 + (alignment != 32))


def test_malformed_files_are_rejected(orc, tmp_path):
    path = tmp_path / "m.gguf"
    make_file(orc, path)
    good = open(path, "rb").read()
    cases = {"magic": b"GGML" + good[4:], "version": good[:4] + struct.pack("<I", 9) + good[8:], "truncated": good[:-100],
             "header cut": good[:40]}
    for what, blob in cases.items():
        p = tmp_path / f"bad_{what.replace(' ', '_')}.gguf"
        p.write_bytes(blob)
        with pytest.raises(gguf.GGUFError):
            gguf.GGUFFile(str(p))
    def header(n_tensors, n_kv, body=b""):
        return b"GGUF" + struct.pack("<IQQ", 3, n_tensors, n_kv) + body

    def s(text):
        return struct.pack("<Q", len(text)) + text

    hostile = {
        "huge counts": header(2 ** 40, 2 ** 40),
        "zero dims": header(1, 0, s(b"t") + struct.pack("<I", 0) + struct.pack("<IQ", 0, 0)),
        "five dims": header(1, 0, s(b"t") + struct.pack("<I", 5) + struct.pack("<5Q", 32, 1, 1, 1, 1) + struct.pack("<IQ", 0, 0)),
        "zero dim": header(1, 0, s(b"t") + struct.pack("<I", 2) + struct.pack("<2Q", 32, 0) + struct.pack("<IQ", 0, 0)),
        "nested array": header(0, 1, s(b"k") + struct.pack("<I", gguf.ARRAY) + struct.pack("<IQ", gguf.ARRAY, 1) + struct.pack("<IQ", gguf.U8, 0)),
        "deep nesting": header(0, 1, s(b"k") + struct.pack("<I", gguf.ARRAY) + struct.pack("<IQ", gguf.ARRAY, 1) * 5000),
        "huge array": header(0, 1, s(b"k") + struct.pack("<I", gguf.ARRAY) + struct.pack("<IQ", gguf.U32, 2 ** 50)),
        "bad array type": header(0, 1, s(b"k") + struct.pack("<I", gguf.ARRAY) + struct.pack("<IQ", 77, 1) + b"\0" * 64),
        "huge string": header(0, 1, struct.pack("<Q", 2 ** 60) + b"abc"),
    }
    for what, blob in hostile.items():
        p = tmp_path / f"hostile_{what.replace(' ', '_')}.gguf"
        p.write_bytes(blob + b"\0" * 64)
        with pytest.raises(gguf.GGUFError):
            gguf.GGUFFile(str(p))
    for dims in ((), (256, 0), (32, 1, 1, 1, 1)):
        with pytest.raises(gguf.GGUFError):
            gguf.tensor_nbytes(2, dims)
    with pytest.raises(gguf.GGUFError):
        gguf.write_gguf(str(tmp_path / "x.gguf"), {}, [("t", (100, 4), 2, np.zeros(10, np.uint8))])   # ragged row
    assert gguf.tensor_nbytes(13, (256, 4)) == 4 * 176                                                # Q5_K
    with pytest.raises(gguf.GGUFError):
        gguf.tensor_nbytes(10, (256, 4))                                                              # Q2_K: not supported


@pytest.mark.gpu
def test_tensors_from_a_file_reach_the_kernels_unchanged(hip, orc, tmp_path):
    path = tmp_path / "m.gguf"
    raw, _ = make_file(orc, path)
    f = gguf.GGUFFile(str(path))
    x = G.seeded_acts(1100, 1, 1024)
    xb = hip.upload(x)
    for name, (t, n, k, blocks) in raw.items():
        w = f.upload(hip, name)
        y = hip.alloc(n * 4)
        hip.quantized_matvec(w, xb, y)
        assert G.max_rel_err(y.download(np.float32, (1, n)), orc.matvec(t, orc.ACT_Q8, blocks, x, n, k)) < 2e-5
    with pytest.raises(gguf.GGUFError):
        f.upload(hip, "output_norm.weight")


class RecordingBackend:
    """Stands in for the device in host-only tests of the loader: remembers what would be uploaded."""

    def __init__(self):
        self.weights, self.vectors = [], []

    def upload_weight(self, qtype, blocks, n, k):
        self.weights.append((qtype, n, k, np.array(blocks)))
        return self.weights[-1]

    def upload(self, arr):
        self.vectors.append(np.array(arr))
        return self.vectors[-1]


DIMS = dict(hidden=256, n_heads=2, n_kv_heads=1, ffn=512, vocab=96, rope_theta=500000.0, eps=1e-5)


def test_model_loader_reads_the_llama_convention(orc, tmp_path):
    from decoderef import write_llama_file
    from openagents_amd.decode import load_gguf_model
    path = tmp_path / "m.gguf"
    host = write_llama_file(orc, path, DIMS, [{"attn_v": "Q6_K"}, {"ffn_down": "Q8_0"}], embd_format="Q5_K", seed=5, norm_types=[0, 1])
    be = RecordingBackend()
    model = load_gguf_model(be, str(path))
    s = model.shape
    assert (s.hidden, s.n_heads, s.n_kv_heads, s.head_dim, s.kv_dim, s.ffn, s.vocab, s.n_layers) == (256, 2, 1, 128, 128, 512, 96, 2)
    assert s.rope_theta == 500000.0
    l0, l1 = model.weights.layers
    assert (l0.wv[0], l0.wv[1], l0.wv[2]) == (orc.Q6_K, 128, 256) and np.array_equal(l0.wv[3].reshape(-1), host["layers"][0]["attn_v"][1].reshape(-1))
    assert (l1.w_down[0], l1.w_down[1], l1.w_down[2]) == (orc.Q8_0, 256, 512)
    assert np.array_equal(l1.attn_norm, host["layers"][1]["attn_norm"])          # stored as F16, widened on load
    assert np.array_equal(model.weights.final_norm, host["final_norm"])
    assert model.weights.lm_head[0] == orc.Q6_K and model.weights.lm_head[1] == 96
    # the embedding table stays on the host: a row is dequantized per token, bit-equal to the oracle's values
    table = orc.dequantize(orc.Q5_K, host["embd"][1], 256)
    for tok in (0, 41, 95):
        assert np.array_equal(model.embedding.row(tok).view(np.uint32), table[tok].view(np.uint32))
    with pytest.raises(IndexError):
        model.embedding.row(96)
    assert not any(w[1] == 96 and w[0] == orc.Q5_K for w in be.weights)           # ... and was not uploaded as a matrix


def test_model_loader_refuses_what_the_step_does_not_compute(orc, tmp_path):
    from decoderef import write_llama_file
    from openagents_amd.decode import load_gguf_model
    be = RecordingBackend()

    def refused(match, **kw):
        path = tmp_path / "bad.gguf"
        write_llama_file(orc, path, kw.pop("dims", DIMS), kw.pop("formats", [{}]), **kw)
        with pytest.raises(gguf.GGUFError, match=match):
            load_gguf_model(be, str(path))

    refused("architecture", extra_metadata={"general.architecture": (gguf.STRING, "qwen2")})
    refused("embedding_length is missing", extra_metadata={"llama.embedding_length": None})
    refused("rotary frequency scaling", extra_metadata={"llama.rope.scaling.type": (gguf.STRING, "linear")})
    refused("rotary frequency scaling", extra_tensors=[("rope_freqs.weight", (64,), 0, np.ones(64, np.float32).view(np.uint8))])
    refused("partial rotary", extra_metadata={"llama.rope.dimension_count": (gguf.U32, 64)})
    refused("biases", extra_tensors=[("blk.0.attn_q.bias", (256,), 0, np.zeros(256, np.float32).view(np.uint8))])
    refused("blk.0.ffn_up.weight is missing", omit=("blk.0.ffn_up.weight",))
    refused("token_embd.weight is missing", omit=("token_embd.weight",))
    refused("metadata implies", extra_metadata={"llama.feed_forward_length": (gguf.U32, 768)})
    refused("not a multiple", extra_metadata={"llama.attention.head_count": (gguf.U32, 3)})
    refused("head layout", extra_metadata={"llama.attention.head_count_kv": (gguf.U32, 0)})
    # per-layer kv-head arrays are accepted when they agree, refused when they differ
    path = tmp_path / "ok.gguf"
    write_llama_file(orc, path, DIMS, [{}, {}], extra_metadata={"llama.attention.head_count_kv": (gguf.ARRAY, (gguf.U32, [1, 1]))})
    assert load_gguf_model(be, str(path)).shape.n_kv_heads == 1
    refused("head_count_kv values differ", formats=[{}, {}], extra_metadata={"llama.attention.head_count_kv": (gguf.ARRAY, (gguf.U32, [1, 2]))})
    # a norm stored in a quantized format is not a vector this loader takes
    q = orc.quantize(orc.Q8_0, np.ones((1, 256), np.float32))
    refused("F32 or F16", omit=("output_norm.weight",), extra_tensors=[("output_norm.weight", (256,), 8, q)])


def test_tied_head_uses_the_embedding_table(orc, tmp_path):
    from decoderef import write_llama_file
    from openagents_amd.decode import load_gguf_model
    path = tmp_path / "tied.gguf"
    host = write_llama_file(orc, path, DIMS, [{}], embd_format="Q8_0", head_format=None)
    be = RecordingBackend()
    model = load_gguf_model(be, str(path))
    assert model.weights.lm_head[0] == orc.Q8_0 and model.weights.lm_head[1:3] == (96, 256)
    assert np.array_equal(model.weights.lm_head[3].reshape(-1), host["embd"][1].reshape(-1))
