"""Reference arithmetic of one Llama-style decode step (numpy in float64 around the oracle's quantized
matvecs) and a writer of small llama-architecture GGUF files with a chosen weight format per tensor.
Test infrastructure only."""
import numpy as np

from openagents_amd import gguf

TYPE_IDS = {"Q4_0": 2, "Q8_0": 8, "Q4_K": 12, "Q5_K": 13, "Q6_K": 14}
MATRICES = {"attn_q": ("hidden", "hidden"), "attn_k": ("kv_dim", "hidden"), "attn_v": ("kv_dim", "hidden"), "attn_output": ("hidden", "hidden"),
            "ffn_gate": ("ffn", "hidden"), "ffn_up": ("ffn", "hidden"), "ffn_down": ("hidden", "ffn")}


def rmsnorm_ref(x, w, eps):
    x = x.astype(np.float64)
    return (x / np.sqrt(np.mean(x * x) + eps) * w).astype(np.float32)


def rope_ref(vec, n_heads, head_dim, pos, theta):
    v = vec.astype(np.float64).reshape(n_heads, head_dim // 2, 2)
    i = np.arange(head_dim // 2)
    ang = pos * theta ** (-2.0 * i / head_dim)
    c, s = np.cos(ang), np.sin(ang)
    out = np.empty_like(v)
    out[:, :, 0] = v[:, :, 0] * c - v[:, :, 1] * s
    out[:, :, 1] = v[:, :, 0] * s + v[:, :, 1] * c
    return out.reshape(-1).astype(np.float32)


def attention_ref(q, kc, vc, n_heads, n_kv, d, n_ctx):
    q = q.astype(np.float64).reshape(n_heads, d)
    k = kc[:n_ctx].astype(np.float64).reshape(n_ctx, n_kv, d)
    v = vc[:n_ctx].astype(np.float64).reshape(n_ctx, n_kv, d)
    out = np.empty((n_heads, d))
    for h in range(n_heads):
        g = h // (n_heads // n_kv)
        s = k[:, g, :] @ q[h] / np.sqrt(d)
        p = np.exp(s - s.max())
        out[h] = (p / p.sum()) @ v[:, g, :]
    return out.reshape(-1).astype(np.float32)


def write_llama_file(orc, path, dims, layer_formats, embd_format="Q4_K", head_format="Q6_K", seed=0, norm_types=None, extra_metadata=None,
                     extra_tensors=(), omit=()):
    """dims: hidden, n_heads, n_kv_heads, ffn, vocab, rope_theta, eps.  layer_formats: one dict per layer,
    tensor stem -> format name (missing stems: Q4_K).  head_format None ties the LM head to token_embd.
    norm_types: per layer 0 (F32) or 1 (F16).  Returns the host copy: {"layers": [{stem: (format, blocks),
    "attn_norm": fp32, "ffn_norm": fp32}], "embd": (format, blocks), "head": (format, blocks), "final_norm"}."""
    rng = np.random.default_rng(seed)
    d = dict(dims)
    d["kv_dim"] = d["hidden"] // d["n_heads"] * d["n_kv_heads"]
    tensors, host = [], {"layers": []}

    def qmat(fmt, n, k, sigma=0.05):
        return orc.quantize(getattr(orc, fmt), rng.standard_normal((n, k), dtype=np.float32) * np.float32(sigma))

    def add(name, dims_, gtype, data):
        if name not in omit:
            tensors.append((name, dims_, gtype, data))

    def add_norm(name, vec, as_f16):
        if as_f16:
            h = vec.astype(np.float16)
            add(name, (vec.size,), 1, h.view(np.uint8))
            return h.astype(np.float32)
        add(name, (vec.size,), 0, vec.view(np.uint8))
        return vec

    host["embd"] = (embd_format, qmat(embd_format, d["vocab"], d["hidden"], 1.0))
    add("token_embd.weight", (d["hidden"], d["vocab"]), TYPE_IDS[embd_format], host["embd"][1])
    for li, fmts in enumerate(layer_formats):
        f16 = bool(norm_types[li]) if norm_types else False
        layer = {}
        layer["attn_norm"] = add_norm(f"blk.{li}.attn_norm.weight", (1 + 0.1 * rng.standard_normal(d["hidden"])).astype(np.float32), f16)
        for stem, (rows, cols) in MATRICES.items():
            fmt = fmts.get(stem, "Q4_K")
            layer[stem] = (fmt, qmat(fmt, d[rows], d[cols]))
            add(f"blk.{li}.{stem}.weight", (d[cols], d[rows]), TYPE_IDS[fmt], layer[stem][1])
        layer["ffn_norm"] = add_norm(f"blk.{li}.ffn_norm.weight", (1 + 0.1 * rng.standard_normal(d["hidden"])).astype(np.float32), f16)
        host["layers"].append(layer)
    host["final_norm"] = add_norm("output_norm.weight", (1 + 0.1 * rng.standard_normal(d["hidden"])).astype(np.float32), False)
    if head_format is None:
        host["head"] = host["embd"]
    else:
        host["head"] = (head_format, qmat(head_format, d["vocab"], d["hidden"]))
        add("output.weight", (d["hidden"], d["vocab"]), TYPE_IDS[head_format], host["head"][1])
    tensors.extend(extra_tensors)
    md = {"general.architecture": (gguf.STRING, "llama"), "general.name": (gguf.STRING, "synthetic"),
          "llama.block_count": (gguf.U32, len(layer_formats)), "llama.embedding_length": (gguf.U32, d["hidden"]),
          "llama.feed_forward_length": (gguf.U32, d["ffn"]), "llama.attention.head_count": (gguf.U32, d["n_heads"]),
          "llama.attention.head_count_kv": (gguf.U32, d["n_kv_heads"]), "llama.rope.freq_base": (gguf.F32, d["rope_theta"]),
          "llama.attention.layer_norm_rms_epsilon": (gguf.F32, d["eps"]), "llama.context_length": (gguf.U32, 8192)}
    md.update(extra_metadata or {})
    md = {k: v for k, v in md.items() if v is not None}
    gguf.write_gguf(str(path), md, tensors)
    return host


def ref_step(orc, dims, host, x, k_caches, v_caches, pos):
    """One token at position pos: x (fp32 embedding) -> logits.  Appends this position's K/V to the fp16
    caches (one [ctx, kv_dim] array per layer) in place."""
    hidden, nh, nkv, ffn, vocab = dims["hidden"], dims["n_heads"], dims["n_kv_heads"], dims["ffn"], dims["vocab"]
    hd = hidden // nh
    kvd = hd * nkv
    theta, eps = dims["rope_theta"], np.float32(dims["eps"])

    def mv(entry, vec, n, k):
        fmt, blocks = entry
        return orc.matvec(getattr(orc, fmt), orc.ACT_Q8, blocks, vec, n, k).reshape(-1)

    x = x.astype(np.float32).copy()
    for li, L in enumerate(host["layers"]):
        xn = rmsnorm_ref(x, L["attn_norm"], eps)
        q = rope_ref(mv(L["attn_q"], xn, hidden, hidden), nh, hd, pos, theta)
        k = rope_ref(mv(L["attn_k"], xn, kvd, hidden), nkv, hd, pos, theta)
        v = mv(L["attn_v"], xn, kvd, hidden)
        k_caches[li][pos], v_caches[li][pos] = k.astype(np.float16), v.astype(np.float16)
        att = attention_ref(q, k_caches[li], v_caches[li], nh, nkv, hd, pos + 1)
        x = x + mv(L["attn_output"], att, hidden, hidden)
        xn = rmsnorm_ref(x, L["ffn_norm"], eps)
        g, u = mv(L["ffn_gate"], xn, ffn, hidden), mv(L["ffn_up"], xn, ffn, hidden)
        act = (g.astype(np.float64) / (1 + np.exp(-g.astype(np.float64))) * u).astype(np.float32)
        x = x + mv(L["ffn_down"], act, hidden, ffn)
    return mv(host["head"], rmsnorm_ref(x, host["final_norm"], eps), vocab, hidden)
