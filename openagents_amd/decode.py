"""One token of a Llama-style decoder on the device: the harness around the quantized matvecs.

Per layer: (residual add +) RMSNorm -> q|k|v in one matvec launch -> rotary + KV-cache append ->
grouped-query attention over the cache -> o -> residual add + RMSNorm -> gate|up in one launch ->
SwiGLU -> down; then the final norm and the LM head.  Every op is a call into the C ABI
(include/psn.h); the whole step can be captured into one HIP graph and replayed.

    python -m openagents_amd.decode [--layers 32] [--ctx 2048] [--steps 20]
    python -m openagents_amd.decode --gguf model.gguf --prompt 1,15043 --new 16

runs the Llama-3-8B-shaped synthetic step (Q4_K projections, Q6_K LM head, random-init weights from
the host quantizers, KV cache pre-filled with fp16 N(0,1)) and prints one JSON record with tokens/s
and the matvec share of the step time.

`load_gguf_model(backend, path)` builds the same step from a model file: the llama-family metadata keys
and tensor names of the GGUF convention, any mix of the five weight formats per tensor (a file whose
attn_v / ffn_down switch format between layers, as the K-quant mixes do, simply gets one launch per
format where matrices share an input).
"""
from __future__ import annotations

import argparse
import json
import sys
import time
from dataclasses import dataclass, field

import numpy as np

from ._ffi import ACT_Q8, Q4_K, Q6_K, Q8_K as Q8_K_ACT
from . import gguf as _gguf
from .backend import DeviceBuffer, HipBackend, QuantizedTensor, act_type_for, actq_layout, row_bytes


@dataclass
class LlamaShape:
    hidden: int = 4096
    n_heads: int = 32
    n_kv_heads: int = 8
    head_dim: int = 128
    ffn: int = 14336
    vocab: int = 128256
    n_layers: int = 32
    rope_theta: float = 500000.0
    eps: float = 1e-5

    @property
    def kv_dim(self) -> int:
        return self.n_kv_heads * self.head_dim


@dataclass
class LayerWeights:
    wq: QuantizedTensor
    wk: QuantizedTensor
    wv: QuantizedTensor
    wo: QuantizedTensor
    w_gate: QuantizedTensor
    w_up: QuantizedTensor
    w_down: QuantizedTensor
    attn_norm: DeviceBuffer
    ffn_norm: DeviceBuffer


@dataclass
class ModelWeights:
    layers: list
    final_norm: DeviceBuffer
    lm_head: QuantizedTensor


def _by_format(ws, ys):
    """Matrices sharing an input, split into the groups one launch can take (same format and K), in
    first-seen order: [([weights], [outputs]), ...]."""
    groups = {}
    for w, y in zip(ws, ys):
        g = groups.setdefault((w.qtype, w.k), ([], []))
        g[0].append(w)
        g[1].append(y)
    return list(groups.values())


class DecodeStep:
    """Owns the activations, KV caches and scratch of one sequence and enqueues one token step."""

    def __init__(self, be: HipBackend, shape: LlamaShape, weights: ModelWeights, max_ctx: int, scheme: int = ACT_Q8,
                 fused_quant: bool = True, fused_norm: bool = True, fused_swiglu: bool = True):
        """fused_quant (scheme Q8): the norm, attention and SwiGLU kernels emit their result already
        quantized, and the matvecs read it with the pre-quantized entry points; otherwise every matvec
        quantizes its fp32 input itself.  fused_norm (with fused_quant): the residual add and the RMSNorm
        run inside the projection that consumes them (psn_qmatvec_norm_multi), the residual stream
        alternating between two buffers.  fused_swiglu (with fused_norm): layers whose gate and up projections
        share a format the fused kernels serve get SwiGLU applied inside the gate|up launch
        (psn_qmatvec_norm_swiglu) and a down projection that quantizes its fp32 input while staging it -- six
        launches instead of seven."""
        self.be, self.shape, self.w, self.max_ctx, self.scheme = be, shape, weights, max_ctx, scheme
        self.fused = fused_quant and scheme == ACT_Q8
        self.fused_norm = self.fused and fused_norm
        s = shape
        self.fused_swiglu = [self.fused_norm and fused_swiglu and lw.w_gate.qtype == lw.w_up.qtype
                             and be.norm_swiglu_supported(lw.w_gate.qtype, s.ffn, s.hidden) for lw in weights.layers]
        if s.n_heads * s.head_dim != s.hidden:
            raise ValueError("n_heads * head_dim must equal hidden")
        f32 = 4
        self.x = be.alloc(s.hidden * f32)            # residual stream
        self.xn = be.alloc(s.hidden * f32)           # normalized copy fed to the matvecs
        self.x2 = be.alloc(s.hidden * f32)           # second residual buffer (norm-fused path)
        self.q = be.alloc(s.hidden * f32)
        self.k = be.alloc(s.kv_dim * f32)
        self.v = be.alloc(s.kv_dim * f32)
        self.attn = be.alloc(s.hidden * f32)
        self.o = be.alloc(s.hidden * f32)
        self.gate = be.alloc(s.ffn * f32)
        self.up = be.alloc(s.ffn * f32)
        self.act = be.alloc(s.ffn * f32)
        self.down = be.alloc(s.hidden * f32)
        self.logits = be.alloc(s.vocab * f32)
        self.attn_ws = be.alloc(s.n_heads * ((max_ctx + 63) // 64) * 130 * f32)
        cache_bytes = max_ctx * s.kv_dim * 2
        self.k_cache = [be.alloc(cache_bytes) for _ in range(s.n_layers)]
        self.v_cache = [be.alloc(cache_bytes) for _ in range(s.n_layers)]
        be.reserve(max(s.hidden, s.ffn), 1)
        self.qkv_launches = [len(_by_format([lw.wq, lw.wk, lw.wv], [0, 1, 2])) for lw in weights.layers]
        self.gate_up_launches = [len(_by_format([lw.w_gate, lw.w_up], [0, 1])) for lw in weights.layers]
        if self.fused:
            # the producers of wo's and w_down's inputs write the activation blocks those matrices read, so the
            # activation type may change from layer to layer; matrices fed by a norm launch of their own
            # (fused_norm off) share its one quantized copy and must agree on the type
            kinds = {act_type_for(t.qtype) for lw in weights.layers for t in (lw.wq, lw.wk, lw.wv, lw.wo, lw.w_gate, lw.w_up, lw.w_down)}
            kinds.add(act_type_for(weights.lm_head.qtype))
            if not self.fused_norm and len(kinds) != 1:
                raise ValueError("with the norm as its own launch, fused quantization needs one activation type for all projections")
            self.act_type = act_type_for(weights.layers[0].wo.qtype)
            self.xq_h = be.alloc(max(int(actq_layout(a, s.hidden, 1).bytes) for a in kinds))
            self.xq_attn = be.alloc(max(int(actq_layout(a, s.hidden, 1).bytes) for a in kinds))
            self.xq_f = be.alloc(max(int(actq_layout(a, s.ffn, 1).bytes) for a in kinds))
            self.rope_tab = be.alloc(s.head_dim * 4)

    @property
    def launches_per_layer(self) -> int:
        """Launches of a layer whose q|k|v and gate|up each share one format."""
        return 7 if self.fused_norm else 9 if self.fused else 10

    @property
    def launches_outside_layers(self) -> int:
        return 2 if self.fused_norm else 3 if self.fused else 2

    @property
    def launches_per_token(self) -> int:
        """Every launch of one step, counting one extra per additional format among q|k|v and gate|up."""
        extra = sum(n - 1 for n in self.qkv_launches) + sum(n - 1 for n in self.gate_up_launches)
        return len(self.w.layers) * self.launches_per_layer + self.launches_outside_layers + extra - sum(self.fused_swiglu)

    def _norm_multi(self, ws, x, delta, norm, h_out, ys):
        """ys = ws . q(rmsnorm(x + delta) * norm): one launch per weight format, each redoing the add and the norm
        from the same x and delta (h_out, written by the first, is a different buffer)."""
        for gi, (gw, gy) in enumerate(_by_format(ws, ys)):
            self.be.quantized_matvec_norm_multi(gw, x, delta, norm, h_out if gi == 0 else None, gy, self.shape.eps)

    def _enqueue_norm_fused(self, pos: int):
        """Seven launches per layer: q|k|v (with add + norm), attention partial, combine, o, gate|up (with
        add + norm), SwiGLU, down -- six where SwiGLU runs inside the gate|up launch.  The residual stream moves
        self.x -> self.x2 -> self.x within a layer."""
        be, s = self.be, self.shape
        be.rope_table(self.rope_tab, s.head_dim, pos, s.rope_theta)
        for li, lw in enumerate(self.w.layers):
            self._norm_multi([lw.wq, lw.wk, lw.wv], self.x, self.down if li > 0 else None, lw.attn_norm, self.x2, [self.q, self.k, self.v])
            be.attention_decode_rope(self.q, self.k, self.v, self.k_cache[li], self.v_cache[li], self.attn_ws, None, self.xq_attn,
                                     act_type_for(lw.wo.qtype), s.n_heads, s.n_kv_heads, s.head_dim, pos, self.rope_tab)
            be.quantized_matvec_q8(lw.wo, self.xq_attn, self.o, 1)
            if self.fused_swiglu[li]:
                be.quantized_matvec_norm_swiglu(lw.w_gate, lw.w_up, self.x2, self.o, lw.ffn_norm, self.x, self.act, s.eps)
                be.quantized_matvec(lw.w_down, self.act, self.down, 1, ACT_Q8)
            else:
                self._norm_multi([lw.w_gate, lw.w_up], self.x2, self.o, lw.ffn_norm, self.x, [self.gate, self.up])
                be.swiglu_q8(self.gate, self.up, None, self.xq_f, act_type_for(lw.w_down.qtype), s.ffn)
                be.quantized_matvec_q8(lw.w_down, self.xq_f, self.down, 1)
        be.quantized_matvec_norm_multi([self.w.lm_head], self.x, self.down, self.w.final_norm, None, [self.logits], s.eps)

    def _enqueue_fused(self, pos: int, matvecs_only: bool):
        be, s, at = self.be, self.shape, self.act_type
        glue = not matvecs_only
        if glue and self.fused_norm:
            return self._enqueue_norm_fused(pos)
        if glue:
            be.rope_table(self.rope_tab, s.head_dim, pos, s.rope_theta)      # once per token
        for li, lw in enumerate(self.w.layers):
            if glue:
                be.add_rmsnorm_q8(self.x, self.down if li > 0 else None, lw.attn_norm, None, self.xq_h, at, s.hidden, s.eps)
            for gw, gy in _by_format([lw.wq, lw.wk, lw.wv], [self.q, self.k, self.v]):
                be.quantized_matvec_q8_multi(gw, self.xq_h, gy, 1)
            if glue:
                be.attention_decode_rope(self.q, self.k, self.v, self.k_cache[li], self.v_cache[li], self.attn_ws, None, self.xq_attn, at,
                                         s.n_heads, s.n_kv_heads, s.head_dim, pos, self.rope_tab)
            be.quantized_matvec_q8(lw.wo, self.xq_attn, self.o, 1)
            if glue:
                be.add_rmsnorm_q8(self.x, self.o, lw.ffn_norm, None, self.xq_h, at, s.hidden, s.eps)
            for gw, gy in _by_format([lw.w_gate, lw.w_up], [self.gate, self.up]):
                be.quantized_matvec_q8_multi(gw, self.xq_h, gy, 1)
            if glue:
                be.swiglu_q8(self.gate, self.up, None, self.xq_f, at, s.ffn)
            be.quantized_matvec_q8(lw.w_down, self.xq_f, self.down, 1)
        if glue:
            be.add_rmsnorm_q8(self.x, self.down, self.w.final_norm, None, self.xq_h, at, s.hidden, s.eps)
        be.quantized_matvec_q8(self.w.lm_head, self.xq_h, self.logits, 1)

    def enqueue(self, pos: int, matvecs_only: bool = False):
        """All launches of one token at position `pos`; self.x holds the token's embedding on entry.
        With matvecs_only the glue ops are skipped (same matvec launches on whatever the buffers hold)."""
        if self.fused:
            return self._enqueue_fused(pos, matvecs_only)
        be, s, sch = self.be, self.shape, self.scheme
        glue = not matvecs_only
        for li, lw in enumerate(self.w.layers):
            if glue:
                be.add_rmsnorm(self.x, self.down if li > 0 else None, lw.attn_norm, self.xn, s.hidden, s.eps)
            for gw, gy in _by_format([lw.wq, lw.wk, lw.wv], [self.q, self.k, self.v]):
                be.quantized_matvec_multi(gw, self.xn, gy, 1, sch)
            if glue:
                be.rope_kv_store(self.q, self.k, self.v, self.k_cache[li], self.v_cache[li], s.n_heads, s.n_kv_heads, s.head_dim, pos, s.rope_theta)
                be.attention_decode(self.q, self.k_cache[li], self.v_cache[li], self.attn_ws, self.attn, s.n_heads, s.n_kv_heads, s.head_dim, pos + 1)
            be.quantized_matvec(lw.wo, self.attn, self.o, 1, sch)
            if glue:
                be.add_rmsnorm(self.x, self.o, lw.ffn_norm, self.xn, s.hidden, s.eps)
            for gw, gy in _by_format([lw.w_gate, lw.w_up], [self.gate, self.up]):
                be.quantized_matvec_multi(gw, self.xn, gy, 1, sch)
            if glue:
                be.swiglu(self.gate, self.up, self.act, s.ffn)
            be.quantized_matvec(lw.w_down, self.act, self.down, 1, sch)
        if glue:
            be.add_rmsnorm(self.x, self.down, self.w.final_norm, self.xn, s.hidden, s.eps)
        be.quantized_matvec(self.w.lm_head, self.xn, self.logits, 1, sch)

    def capture(self, pos: int, matvecs_only: bool = False):
        self.be.begin_capture()
        self.enqueue(pos, matvecs_only)
        return self.be.end_capture()

    def matvec_bytes(self) -> float:
        """Algorithmic bytes of one step's matvecs (GGUF weight bytes + fp32 in/out vectors)."""
        total = 0.0
        for lw in self.w.layers:
            for t in (lw.wq, lw.wk, lw.wv, lw.wo, lw.w_gate, lw.w_up, lw.w_down):
                total += t.n * row_bytes(t.qtype, t.k) + 4 * t.n
            total += 4 * (3 * self.shape.hidden + self.shape.ffn)
        t = self.w.lm_head
        return total + t.n * row_bytes(t.qtype, t.k) + 4 * (t.n + t.k)


def synthetic_weights(be: HipBackend, shape: LlamaShape, seed: int = 0, unique_layers: int = 1, head_rows_unique: int = 16032,
                      keep_host: dict | None = None) -> ModelWeights:
    """Random-init weights of the given architecture: fp32 N(0, 0.02) quantized on the host by the
    library's reference quantizers (Q4_K projections, Q6_K LM head).  `unique_layers` layers are generated
    and uploaded round-robin into n_layers distinct device allocations; the LM head is `head_rows_unique`
    unique rows tiled.  With `keep_host` the unique host blocks are left in that dict (name -> uint8 array)."""
    from . import quantize
    rng = np.random.default_rng(seed)
    s = shape

    def qmat(n, k, qtype=Q4_K):
        w = (rng.standard_normal((n, k), dtype=np.float32) * np.float32(0.02))
        return (quantize.quantize_q4_K(w) if qtype == Q4_K else quantize.quantize_q6_K(w))

    protos = []
    for _ in range(unique_layers):
        protos.append({"wq": qmat(s.hidden, s.hidden), "wk": qmat(s.kv_dim, s.hidden), "wv": qmat(s.kv_dim, s.hidden),
                       "wo": qmat(s.hidden, s.hidden), "w_gate": qmat(s.ffn, s.hidden), "w_up": qmat(s.ffn, s.hidden),
                       "w_down": qmat(s.hidden, s.ffn)})
    dims = {"wq": (s.hidden, s.hidden), "wk": (s.kv_dim, s.hidden), "wv": (s.kv_dim, s.hidden), "wo": (s.hidden, s.hidden),
            "w_gate": (s.ffn, s.hidden), "w_up": (s.ffn, s.hidden), "w_down": (s.hidden, s.ffn)}
    layers = []
    for li in range(s.n_layers):
        p = protos[li % unique_layers]
        t = {name: be.upload_weight(Q4_K, p[name], *dims[name]) for name in dims}
        layers.append(LayerWeights(**t, attn_norm=be.upload(np.ones(s.hidden, np.float32)), ffn_norm=be.upload(np.ones(s.hidden, np.float32))))
    uniq = min(head_rows_unique, s.vocab)
    head = qmat(uniq, s.hidden, Q6_K)
    reps = -(-s.vocab // uniq)
    head_full = np.tile(head, (reps, 1))[:s.vocab]
    if keep_host is not None:
        for i, p in enumerate(protos):
            keep_host.update({f"layer{i}.{name}": blk for name, blk in p.items()})
        keep_host["lm_head"] = head
    return ModelWeights(layers, be.upload(np.ones(s.hidden, np.float32)), be.upload_weight(Q6_K, head_full, s.vocab, s.hidden))


class TokenEmbedding:
    """The embedding table of a model file, left on the host in the file's mapping: one row is
    dequantized per token (psn_dequantize_rows), which is all a decode step reads of it."""

    def __init__(self, gf: "_gguf.GGUFFile", name: str = "token_embd.weight"):
        t = gf.tensors[name]
        self.info, self.bytes = t, gf.data(name)
        self.hidden, self.vocab = t.k, t.n
        self.row_nbytes = t.nbytes // t.n

    def row(self, token: int) -> np.ndarray:
        if not 0 <= token < self.vocab:
            raise IndexError(f"token {token} outside the vocabulary of {self.vocab}")
        raw = self.bytes[token * self.row_nbytes:(token + 1) * self.row_nbytes]
        if self.info.ggml_type == 0:
            return np.array(raw.view(np.float32))
        if self.info.ggml_type == 1:
            return raw.view(np.float16).astype(np.float32)
        from . import quantize
        return quantize.dequantize(self.info.ggml_type, raw, self.hidden)[0]


@dataclass
class GGUFModel:
    shape: LlamaShape
    weights: ModelWeights
    embedding: TokenEmbedding
    file: "_gguf.GGUFFile"


_LAYER_TENSORS = {"wq": "attn_q", "wk": "attn_k", "wv": "attn_v", "wo": "attn_output", "w_gate": "ffn_gate", "w_up": "ffn_up", "w_down": "ffn_down"}


def load_gguf_model(be: HipBackend, path: str) -> GGUFModel:
    """Read a llama-architecture GGUF file into device weights.

    Metadata: general.architecture = "llama", llama.{block_count, embedding_length, feed_forward_length,
    attention.head_count, attention.head_count_kv (default head_count), attention.key_length (default
    embedding_length / head_count), attention.layer_norm_rms_epsilon (default 1e-5), rope.freq_base
    (default 10000)}.  Tensors: token_embd, output_norm, output (absent = tied to token_embd),
    blk.N.{attn_norm, attn_q, attn_k, attn_v, attn_output, ffn_norm, ffn_gate, ffn_up, ffn_down}.weight;
    projections in any of Q4_0 / Q8_0 / Q4_K / Q5_K / Q6_K, norms in F32 or F16.  What this step does not
    compute is refused rather than ignored: another architecture, projection biases, rotary scaling."""
    gf = _gguf.GGUFFile(path)
    md = gf.metadata
    arch = md.get("general.architecture")
    if arch != "llama":
        raise _gguf.GGUFError(f"general.architecture = {arch!r}: only the llama layer structure is implemented")

    def need(key):
        if f"llama.{key}" not in md:
            raise _gguf.GGUFError(f"metadata key llama.{key} is missing")
        return md[f"llama.{key}"]

    hidden, n_heads = int(need("embedding_length")), int(need("attention.head_count"))
    n_kv = md.get("llama.attention.head_count_kv", n_heads)
    if isinstance(n_kv, list):
        if len(set(n_kv)) != 1:
            raise _gguf.GGUFError("per-layer head_count_kv values differ")
        n_kv = n_kv[0]
    if n_heads <= 0 or hidden % n_heads:
        raise _gguf.GGUFError(f"embedding_length {hidden} is not a multiple of head_count {n_heads}")
    head_dim = int(md.get("llama.attention.key_length", hidden // n_heads))
    scaling = md.get("llama.rope.scaling.type", "none")
    if scaling not in ("none", "") or "rope_freqs.weight" in gf.tensors:
        raise _gguf.GGUFError("rotary frequency scaling (rope.scaling / rope_freqs) is not implemented")
    if int(md.get("llama.rope.dimension_count", head_dim)) != head_dim:
        raise _gguf.GGUFError("partial rotary embedding (rope.dimension_count < head size) is not implemented")
    if "token_embd.weight" not in gf.tensors:
        raise _gguf.GGUFError("tensor token_embd.weight is missing")
    emb = TokenEmbedding(gf)
    head_name = "output.weight" if "output.weight" in gf.tensors else "token_embd.weight"
    shape = LlamaShape(hidden=hidden, n_heads=n_heads, n_kv_heads=int(n_kv), head_dim=head_dim, ffn=int(need("feed_forward_length")),
                       vocab=gf.tensors[head_name].n, n_layers=int(need("block_count")),
                       rope_theta=float(md.get("llama.rope.freq_base", 10000.0)), eps=float(md.get("llama.attention.layer_norm_rms_epsilon", 1e-5)))
    if n_heads * head_dim != hidden or shape.n_kv_heads <= 0 or n_heads % shape.n_kv_heads:
        raise _gguf.GGUFError(f"head layout {n_heads} x {head_dim} (kv {shape.n_kv_heads}) does not match embedding_length {hidden}")
    if emb.hidden != hidden:
        raise _gguf.GGUFError(f"token_embd rows hold {emb.hidden} values, embedding_length is {hidden}")

    def matrix(name, n, k):
        if name not in gf.tensors:
            raise _gguf.GGUFError(f"tensor {name} is missing")
        t = gf.tensors[name]
        if (t.n, t.k) != (n, k):
            raise _gguf.GGUFError(f"tensor {name} is [{t.n}, {t.k}], the metadata implies [{n}, {k}]")
        return gf.upload(be, name)

    def vector(name, n):
        if name not in gf.tensors:
            raise _gguf.GGUFError(f"tensor {name} is missing")
        t = gf.tensors[name]
        if t.ggml_type not in (0, 1) or (t.n, t.k) != (1, n):
            raise _gguf.GGUFError(f"tensor {name}: want {n} F32 or F16 values")
        raw = gf.data(name)
        return be.upload(np.array(raw.view(np.float32)) if t.ggml_type == 0 else raw.view(np.float16).astype(np.float32))

    dims = {"wq": (hidden, hidden), "wk": (shape.kv_dim, hidden), "wv": (shape.kv_dim, hidden), "wo": (hidden, hidden),
            "w_gate": (shape.ffn, hidden), "w_up": (shape.ffn, hidden), "w_down": (hidden, shape.ffn)}
    layers = []
    for li in range(shape.n_layers):
        for bias in ("attn_q", "attn_k", "attn_v", "attn_output"):
            if f"blk.{li}.{bias}.bias" in gf.tensors:
                raise _gguf.GGUFError(f"blk.{li}.{bias}.bias: projection biases are not implemented")
        t = {field_: matrix(f"blk.{li}.{stem}.weight", *dims[field_]) for field_, stem in _LAYER_TENSORS.items()}
        layers.append(LayerWeights(**t, attn_norm=vector(f"blk.{li}.attn_norm.weight", hidden), ffn_norm=vector(f"blk.{li}.ffn_norm.weight", hidden)))
    weights = ModelWeights(layers, vector("output_norm.weight", hidden), matrix(head_name, shape.vocab, hidden))
    return GGUFModel(shape, weights, emb, gf)


def greedy_tokens(model: GGUFModel, step: "DecodeStep", prompt, n_new: int):
    """Feed `prompt` (token ids) one position at a time from an empty cache, then extend it by n_new
    arg-max tokens.  Returns (all tokens, the logits that chose the last one; with n_new = 0 the logits after
    the prompt).  A plain host loop: embedding row to the device, one step's launches, logits back."""
    tokens = [int(t) for t in prompt]
    if not tokens:
        raise ValueError("need at least one prompt token")
    if len(tokens) + n_new > step.max_ctx:
        raise ValueError(f"{len(tokens)} prompt + {n_new} new tokens exceed the context of {step.max_ctx}")
    pos = 0
    while True:
        step.x.upload(model.embedding.row(tokens[pos]))
        step.enqueue(pos)
        if pos == len(tokens) - 1:                     # the newest token: its logits choose the next one
            logits = step.logits.download(np.float32, (model.shape.vocab,))
            if n_new == 0:
                break
            tokens.append(int(np.argmax(logits)))
            n_new -= 1
            if n_new == 0:
                break
        pos += 1
    return tokens, logits


def attention_sweep(be: HipBackend, contexts, samples: int = 9, n_heads: int = 32, n_kv_heads: int = 8, head_dim: int = 128):
    """Time psn_attention_decode_rope (two launches) for a token at the last position of each context length, over
    enough distinct KV caches that no launch finds its rows in a cache: microseconds per call and the rate at which
    the K and V rows (fp16) are read."""
    from . import records as R
    rng = np.random.default_rng(0)
    row = n_kv_heads * head_dim
    q, k, v = (be.upload(rng.standard_normal(n, dtype=np.float32)) for n in (n_heads * head_dim, row, row))
    out_q = be.alloc(int(actq_layout(Q8_K_ACT, n_heads * head_dim, 1).bytes))
    tab = be.alloc(head_dim * 4)
    rows = []
    for ctx in contexts:
        nbytes = ctx * row * 2
        copies = max(2, min(8, int(700e6 // (2 * nbytes)) + 1))
        block = rng.standard_normal((min(ctx, 4096), row), dtype=np.float32).astype(np.float16)
        caches = []
        for _ in range(2 * copies):
            buf = be.alloc(nbytes)
            for off in range(0, ctx, block.shape[0]):
                buf.upload(block[:min(block.shape[0], ctx - off)], off * row * 2)
            caches.append(buf)
        ws = be.alloc(n_heads * ((ctx + 63) // 64) * 130 * 4)
        be.rope_table(tab, head_dim, ctx - 1, 500000.0)
        be.begin_capture()
        for i in range(copies):
            be.attention_decode_rope(q, k, v, caches[2 * i], caches[2 * i + 1], ws, None, out_q, Q8_K_ACT, n_heads, n_kv_heads, head_dim, ctx - 1, tab)
        g = be.end_capture()
        st = R.stats(R.time_graph(be, g, copies, samples))
        be.destroy_graph(g)
        rows.append({"context": ctx, "us": round(st["median_us"], 2), "kv_MB": round(2 * nbytes / 1e6, 1),
                     "kv_TBps": round(2 * nbytes / st["median_us"] / 1e6, 2), "heads": f"{n_heads}/{n_kv_heads}"})
        for b in caches + [ws]:
            b.free()
    return rows


def main(argv=None):
    ap = argparse.ArgumentParser()
    ap.add_argument("--layers", type=int, default=32)
    ap.add_argument("--ctx", type=int, default=2048)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--seed", type=int, default=0)
    ap.add_argument("--unfused", action="store_true", help="every matvec quantizes its own fp32 input")
    ap.add_argument("--separate-norm", action="store_true", help="RMSNorm as its own launch instead of inside the consuming projection")
    ap.add_argument("--separate-swiglu", action="store_true", help="SwiGLU as its own launch instead of inside the gate|up projection")
    ap.add_argument("--gguf", help="decode greedily from this llama-architecture model file instead of timing the synthetic step")
    ap.add_argument("--prompt", default="1", help="with --gguf: comma-separated prompt token ids (no tokenizer is part of this library)")
    ap.add_argument("--new", type=int, default=16, help="with --gguf: tokens to generate")
    ap.add_argument("--attention-sweep", help="comma-separated context lengths: time the attention of one layer (rotary, cache append, "
                                              "split kernel, combine) at each and exit")
    args = ap.parse_args(argv)
    be = HipBackend(0)
    if args.attention_sweep:
        print(json.dumps({"attention_sweep": attention_sweep(be, [int(c) for c in args.attention_sweep.split(",")], args.steps)}))
        return 0
    if args.gguf:
        t0 = time.time()
        model = load_gguf_model(be, args.gguf)
        load_s = time.time() - t0
        prompt = [int(t) for t in args.prompt.split(",")]
        step = DecodeStep(be, model.shape, model.weights, min(args.ctx, max(len(prompt) + args.new, 1)),
                          fused_quant=not args.unfused, fused_norm=not args.separate_norm, fused_swiglu=not args.separate_swiglu)
        t0 = time.time()
        tokens, logits = greedy_tokens(model, step, prompt, args.new)
        wall = time.time() - t0
        s = model.shape
        print(json.dumps({"file": args.gguf, "tokens": tokens, "prompt_tokens": len(prompt), "new_tokens": len(tokens) - len(prompt),
                          "steps_per_s_host_loop": round((len(tokens) - 1) / wall, 1) if wall > 0 and len(tokens) > 1 else None,
                          "launches_per_token": step.launches_per_token, "load_s": round(load_s, 2),
                          "config": {"layers": s.n_layers, "hidden": s.hidden, "heads": s.n_heads, "kv_heads": s.n_kv_heads, "ffn": s.ffn,
                                     "vocab": s.vocab, "rope_theta": s.rope_theta, "eps": s.eps},
                          "formats": sorted({_gguf.GGML_TYPES[t.qtype][2] for lw in model.weights.layers
                                             for t in (lw.wq, lw.wk, lw.wv, lw.wo, lw.w_gate, lw.w_up, lw.w_down)} |
                                            {_gguf.GGML_TYPES[model.weights.lm_head.qtype][2]}),
                          "logits_finite": bool(np.all(np.isfinite(logits))),
                          "note": "eager launches from a Python loop (host-bound); the timed figure is the graph replay of the synthetic step"}))
        return 0
    shape = LlamaShape(n_layers=args.layers)
    t0 = time.time()
    weights = synthetic_weights(be, shape, args.seed)
    step = DecodeStep(be, shape, weights, args.ctx, fused_quant=not args.unfused, fused_norm=not args.separate_norm, fused_swiglu=not args.separate_swiglu)
    rng = np.random.default_rng(args.seed + 1)
    pos = args.ctx - 1
    kv = rng.standard_normal((pos, shape.kv_dim), dtype=np.float32).astype(np.float16)
    for li in range(shape.n_layers):                 # cache pre-filled up to the position being decoded
        step.k_cache[li].upload(kv)
        step.v_cache[li].upload(kv)
    x0 = rng.standard_normal(shape.hidden, dtype=np.float32)
    setup_s = time.time() - t0

    def timed(graph):
        for _ in range(args.warmup):
            step.x.upload(x0)
            be.launch_graph(graph)
        be.sync()
        e0, e1 = be.event(), be.event()
        be.record(e0)
        for _ in range(args.steps):
            be.launch_graph(graph)
        be.record(e1)
        us = be.elapsed_us(e0, e1) / args.steps
        be.destroy_event(e0)
        be.destroy_event(e1)
        return us

    full = step.capture(pos)
    mv = step.capture(pos, matvecs_only=True)
    t_full, t_mv = timed(full), timed(mv)
    step.x.upload(x0)
    be.launch_graph(full)
    logits = step.logits.download(np.float32, (shape.vocab,))
    mbytes = step.matvec_bytes()
    rec = {"metric": "decode tokens/s (synthetic Llama-3-8B shape, batch 1)", "tokens_per_s": round(1e6 / t_full, 1),
           "ms_per_token": round(t_full / 1e3, 4), "matvec_ms": round(t_mv / 1e3, 4), "matvec_share": round(t_mv / t_full, 4),
           "matvec_GBps": round(mbytes / t_mv / 1e3, 1), "matvec_bytes_per_token": int(mbytes),
           "hbm_peak_GBps": 8000.0, "matvec_frac_of_hbm_peak": round(mbytes / t_mv / 1e3 / 8000.0, 4),
           "config": {"layers": shape.n_layers, "hidden": shape.hidden, "heads": shape.n_heads, "kv_heads": shape.n_kv_heads,
                      "ffn": shape.ffn, "vocab": shape.vocab, "context": args.ctx, "weights": "Q4_K projections, Q6_K LM head",
                      "activation_scheme": "Q8 (Q8_K blocks, " + ("written by the producing kernel)" if step.fused else "quantized inside the matvec launch)"),
                      "launches_per_token": step.launches_per_token, "graph_replay": True},
           "data": "synthetic random-init weights (one unique layer copied to every layer's own allocation), fp16 N(0,1) KV cache",
           "logits_finite": bool(np.all(np.isfinite(logits))), "steps": args.steps, "setup_s": round(setup_s, 1),
           "not_measured": ["sampling", "tokenizer", "host loop"]}
    print(json.dumps(rec))
    return 0


if __name__ == "__main__":
    sys.exit(main())
