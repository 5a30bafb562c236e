"""One token of a Llama-style decoder on the device: the harness around the quantized matvecs.

Per layer: (residual add +) RMSNorm -> q|k|v in one matvec launch -> rotary + KV-cache append ->
grouped-query attention over the cache -> o -> residual add + RMSNorm -> gate|up in one launch ->
SwiGLU -> down; then the final norm and the LM head.  Every op is a call into the C ABI
(include/psn.h); the whole step can be captured into one HIP graph and replayed.

    python -m openagents_amd.decode [--layers 32] [--ctx 2048] [--steps 20]

runs the Llama-3-8B-shaped synthetic step (Q4_K projections, Q6_K LM head, random-init weights from
the host quantizers, KV cache pre-filled with fp16 N(0,1)) and prints one JSON record with tokens/s
and the matvec share of the step time.
"""
from __future__ import annotations

import argparse
import json
import sys
import time
from dataclasses import dataclass, field

import numpy as np

from ._ffi import ACT_Q8, Q4_K, Q6_K
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


class DecodeStep:
    """Owns the activations, KV caches and scratch of one sequence and enqueues one token step."""

    def __init__(self, be: HipBackend, shape: LlamaShape, weights: ModelWeights, max_ctx: int, scheme: int = ACT_Q8,
                 fused_quant: bool = True, fused_norm: bool = True):
        """fused_quant (scheme Q8): the norm, attention and SwiGLU kernels emit their result already
        quantized, and the matvecs read it with the pre-quantized entry points; otherwise every matvec
        quantizes its fp32 input itself.  fused_norm (with fused_quant): the residual add and the RMSNorm
        run inside the projection that consumes them (psn_qmatvec_norm_multi), the residual stream
        alternating between two buffers."""
        self.be, self.shape, self.w, self.max_ctx, self.scheme = be, shape, weights, max_ctx, scheme
        self.fused = fused_quant and scheme == ACT_Q8
        self.fused_norm = self.fused and fused_norm
        s = shape
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
        if self.fused:
            l0 = weights.layers[0]
            kinds = {act_type_for(t.qtype) for t in (l0.wq, l0.wo, l0.w_gate, l0.w_down, weights.lm_head)}
            if len(kinds) != 1:
                raise ValueError("fused quantization needs one activation type for all projections")
            self.act_type = kinds.pop()
            self.xq_h = be.alloc(int(actq_layout(self.act_type, s.hidden, 1).bytes))
            self.xq_attn = be.alloc(int(actq_layout(self.act_type, s.hidden, 1).bytes))
            self.xq_f = be.alloc(int(actq_layout(self.act_type, s.ffn, 1).bytes))
            self.rope_tab = be.alloc(s.head_dim * 4)

    @property
    def launches_per_layer(self) -> int:
        return 7 if self.fused_norm else 9 if self.fused else 10

    @property
    def launches_outside_layers(self) -> int:
        return 2 if self.fused_norm else 3 if self.fused else 2

    def _enqueue_norm_fused(self, pos: int):
        """Seven launches per layer: q|k|v (with add + norm), attention partial, combine, o, gate|up (with
        add + norm), SwiGLU, down.  The residual stream moves self.x -> self.x2 -> self.x within a layer."""
        be, s, at = self.be, self.shape, self.act_type
        be.rope_table(self.rope_tab, s.head_dim, pos, s.rope_theta)
        for li, lw in enumerate(self.w.layers):
            be.quantized_matvec_norm_multi([lw.wq, lw.wk, lw.wv], self.x, self.down if li > 0 else None, lw.attn_norm, self.x2,
                                           [self.q, self.k, self.v], s.eps)
            be.attention_decode_rope(self.q, self.k, self.v, self.k_cache[li], self.v_cache[li], self.attn_ws, None, self.xq_attn, at,
                                     s.n_heads, s.n_kv_heads, s.head_dim, pos, self.rope_tab)
            be.quantized_matvec_q8(lw.wo, self.xq_attn, self.o, 1)
            be.quantized_matvec_norm_multi([lw.w_gate, lw.w_up], self.x2, self.o, lw.ffn_norm, self.x, [self.gate, self.up], s.eps)
            be.swiglu_q8(self.gate, self.up, None, self.xq_f, at, s.ffn)
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
            be.quantized_matvec_q8_multi([lw.wq, lw.wk, lw.wv], self.xq_h, [self.q, self.k, self.v], 1)
            if glue:
                be.attention_decode_rope(self.q, self.k, self.v, self.k_cache[li], self.v_cache[li], self.attn_ws, None, self.xq_attn, at,
                                         s.n_heads, s.n_kv_heads, s.head_dim, pos, self.rope_tab)
            be.quantized_matvec_q8(lw.wo, self.xq_attn, self.o, 1)
            if glue:
                be.add_rmsnorm_q8(self.x, self.o, lw.ffn_norm, None, self.xq_h, at, s.hidden, s.eps)
            be.quantized_matvec_q8_multi([lw.w_gate, lw.w_up], self.xq_h, [self.gate, self.up], 1)
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
            be.quantized_matvec_multi([lw.wq, lw.wk, lw.wv], self.xn, [self.q, self.k, self.v], 1, sch)
            if glue:
                be.rope_kv_store(self.q, self.k, self.v, self.k_cache[li], self.v_cache[li], s.n_heads, s.n_kv_heads, s.head_dim, pos, s.rope_theta)
                be.attention_decode(self.q, self.k_cache[li], self.v_cache[li], self.attn_ws, self.attn, s.n_heads, s.n_kv_heads, s.head_dim, pos + 1)
            be.quantized_matvec(lw.wo, self.attn, self.o, 1, sch)
            if glue:
                be.add_rmsnorm(self.x, self.o, lw.ffn_norm, self.xn, s.hidden, s.eps)
            be.quantized_matvec_multi([lw.w_gate, lw.w_up], self.xn, [self.gate, self.up], 1, sch)
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


def main(argv=None):
    ap = argparse.ArgumentParser()
    ap.add_argument("--layers", type=int, default=32)
    ap.add_argument("--ctx", type=int, default=2048)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--seed", type=int, default=0)
    ap.add_argument("--unfused", action="store_true", help="every matvec quantizes its own fp32 input")
    ap.add_argument("--separate-norm", action="store_true", help="RMSNorm as its own launch instead of inside the consuming projection")
    args = ap.parse_args(argv)
    be = HipBackend(0)
    shape = LlamaShape(n_layers=args.layers)
    t0 = time.time()
    weights = synthetic_weights(be, shape, args.seed)
    step = DecodeStep(be, shape, weights, args.ctx, fused_quant=not args.unfused, fused_norm=not args.separate_norm)
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
                      "launches_per_token": shape.n_layers * step.launches_per_layer + step.launches_outside_layers, "graph_replay": True},
           "data": "synthetic random-init weights (one unique layer copied to every layer's own allocation), fp16 N(0,1) KV cache",
           "logits_finite": bool(np.all(np.isfinite(logits))), "steps": args.steps, "setup_s": round(setup_s, 1),
           "not_measured": ["sampling", "tokenizer", "host loop"]}
    print(json.dumps(rec))
    return 0


if __name__ == "__main__":
    sys.exit(main())
