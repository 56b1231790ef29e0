"""Plain, slow implementation of the Qwen3 dense decoder, written from the reference's formulas.

Whole sequences, no cache, one function per part, NumPy only.  It shares no code with the
engine: the engine is tested against it.  Citations are paths inside the reference
checkout (exec-software/exec-beholdd).

Precision follows the reference's CPU device: activations are float32; the sum of squares of
RMSNorm, the attention dot products and value sums, and the rotation angles are float64
and rounded to float32 where the reference rounds them.  One deliberate difference: matrix
products accumulate in float64 and are rounded once (the reference accumulates in float32,
crates/beholdd-backend/src/cpu.rs:206-211), so that this file is the more exact of the two.
"""

from __future__ import annotations

import json
import math
import os

import numpy as np

F32 = np.float32
F64 = np.float64


# ----------------------------------------------------------------------------------------
# parts
# ----------------------------------------------------------------------------------------

def rmsnorm(x, w, eps):
    """y = (x * inv) * w with inv = 1/sqrt(mean(x^2) + eps); the weight is a plain multiplier.

    crates/beholdd-kernel/src/vecops.rs:54-64: sum of squares and the inverse in f64, the
    inverse rounded to f32, then `x[i] * inv * w[i]` in f32 (left to right).
    `x` is [..., n]; `w` is [n] or None.
    """
    x = np.asarray(x, dtype=F32)
    ss = (x.astype(F64) ** 2).sum(axis=-1, keepdims=True)
    inv = (1.0 / np.sqrt(ss / x.shape[-1] + F64(F32(eps)))).astype(F32)
    y = x * inv
    if w is not None:
        y = y * np.asarray(w, dtype=F32)
    return y.astype(F32)


def softmax(v):
    """Stable softmax over the last axis in f32; -inf gives exactly 0; an all -inf row gives zeros.

    crates/beholdd-kernel/src/vecops.rs:70-87: m = max, e = exp(v - m), p = e * (1/sum).
    """
    v = np.asarray(v, dtype=F32)
    m = v.max(axis=-1, keepdims=True)
    dead = ~np.isfinite(m)
    safe_m = np.where(dead, F32(0), m)
    with np.errstate(invalid="ignore"):
        e = np.where(np.isfinite(v), np.exp((v - safe_m).astype(F32)), F32(0)).astype(F32)
    s = e.sum(axis=-1, keepdims=True, dtype=F32)
    with np.errstate(divide="ignore", invalid="ignore"):
        p = e * (F32(1) / s)
    return np.where(dead, F32(0), p).astype(F32)


def silu(x):
    """x / (1 + exp(-x)); crates/beholdd-kernel/src/vecops.rs:91-93."""
    x = np.asarray(x, dtype=F32)
    return (x / (F32(1) + np.exp(-x))).astype(F32)


def swiglu(gate, up, limit=0.0):
    """silu(gate) * up; a positive `limit` clamps gate from above only and up both ways.

    crates/beholdd-kernel/src/vecops.rs:101-110.  Qwen3 uses limit = 0 (no clamp),
    crates/beholdd-model/src/qwen3moe/forward.rs:1288.
    """
    gate = np.asarray(gate, dtype=F32)
    up = np.asarray(up, dtype=F32)
    if limit > 0:
        gate = np.minimum(gate, F32(limit))
        up = np.clip(up, F32(-limit), F32(limit))
    return (silu(gate) * up).astype(F32)


def rope_frequencies(theta, dim):
    """freq[i] = 1 / theta^(2i/dim) for i < dim/2, in f64.

    crates/beholdd-model/src/qwen3moe/forward.rs:1844-1851.
    """
    half = dim // 2
    return np.array([1.0 / math.pow(float(theta), (2 * i) / dim) for i in range(half)], dtype=F64)


def rope_cos_sin(freqs, position):
    """cos/sin of position*freq, the angle in f64, the results stored as f32.

    crates/beholdd-model/src/qwen3moe/forward.rs:1853-1868.
    """
    angle = F64(position) * np.asarray(freqs, dtype=F64)
    return np.cos(angle).astype(F32), np.sin(angle).astype(F32)


def rope_split_half(x, cos, sin, inverse=False):
    """Pairs are (x[i], x[i + n/2]): x[i]' = a*c - b*s, x[i+n/2]' = a*s + b*c.

    crates/beholdd-kernel/src/vecops.rs:186-197.  `x` is [..., n]; cos, sin are [n/2].
    """
    x = np.asarray(x, dtype=F32)
    half = x.shape[-1] // 2
    a, b = x[..., :half], x[..., half:]
    c = np.asarray(cos, dtype=F32)
    s = np.asarray(sin, dtype=F32) * (F32(-1) if inverse else F32(1))
    return np.concatenate([a * c - b * s, a * s + b * c], axis=-1).astype(F32)


def rope_interleaved(x, cos, sin, inverse=False):
    """Adjacent pairs (x[2i], x[2i+1]); NOT what Qwen3 uses.  Kept so that a test can show
    that the two conventions differ (crates/beholdd-kernel/src/vecops.rs:167-176)."""
    x = np.asarray(x, dtype=F32).copy()
    c = np.asarray(cos, dtype=F32)
    s = np.asarray(sin, dtype=F32) * (F32(-1) if inverse else F32(1))
    a, b = x[..., 0::2].copy(), x[..., 1::2].copy()
    x[..., 0::2] = a * c - b * s
    x[..., 1::2] = a * s + b * c
    return x


def linear(x, w):
    """y[r] = sum_i W[r, i] * x[i] for W stored [rows=out, cols=in]; no bias.

    crates/beholdd-backend/src/lib.rs:178, crates/beholdd-backend/src/cpu.rs:206-211.
    Accumulated in f64 here and rounded once to f32.
    """
    return (np.asarray(x, dtype=F64) @ np.asarray(w, dtype=F64).T).astype(F32)


def causal_attention(q, k, v, n_heads, n_kv_heads, head_dim, scale, query_start=0):
    """Causal grouped-query attention.

    q is [Tq, n_heads*head_dim] laid [t][head][d]; k, v are [Tk, n_kv_heads*head_dim].
    Query t stands at absolute position query_start + t and sees keys 0..=that position (the
    mask is the loop bound); head h reads kv head h // (n_heads // n_kv_heads); the dot
    product and the scale are f64, the score is rounded to f32, softmax is f32, and the
    value sum is f64 rounded to f32.
    crates/beholdd-backend/src/cpu.rs:585-691 (whole chunk) and :693-837 (over a cache).
    """
    q = np.asarray(q, dtype=F32)
    k = np.asarray(k, dtype=F32)
    v = np.asarray(v, dtype=F32)
    tq, tk = q.shape[0], k.shape[0]
    group = n_heads // n_kv_heads
    qh = q.reshape(tq, n_heads, head_dim)
    kh = k.reshape(tk, n_kv_heads, head_dim)
    vh = v.reshape(tk, n_kv_heads, head_dim)
    out = np.zeros((tq, n_heads, head_dim), dtype=F32)
    assert query_start + tq <= tk, "a query may not stand beyond the keys"
    some = 256        # queries taken together (the arithmetic of each is the same as if it stood alone)
    for h in range(n_heads):
        kvh = h // group
        keys, values = kh[:, kvh, :].astype(F64), vh[:, kvh, :].astype(F64)
        for t in range(0, tq, some):
            last = min(t + some, tq)
            visible = query_start + last                       # keys that the last of these queries sees
            dots = qh[t:last, h, :].astype(F64) @ keys[:visible].T
            scores = (dots * F64(F32(scale))).astype(F32)
            # the reference's mask is the loop bound: a key beyond a query's position takes no part
            beyond = np.arange(visible)[None, :] > (query_start + np.arange(t, last))[:, None]
            scores[beyond] = -np.inf
            p = softmax(scores)
            out[t:last, h, :] = (p.astype(F64) @ values[:visible]).astype(F32)
    return out.reshape(tq, n_heads * head_dim)


def embed(tokens, table):
    """hidden[t] = table[token[t]], widened to f32, no scaling.

    crates/beholdd-model/src/qwen3moe/forward.rs:954-972.
    """
    table = np.asarray(table)
    tokens = np.asarray(tokens, dtype=np.int64)
    assert tokens.min() >= 0 and tokens.max() < table.shape[0]
    return table[tokens].astype(F32)


def greedy_token(logits):
    """argmax with strict '>': ties go to the lowest id; a non-finite logit is an error.

    crates/beholdd-model/src/qwen3moe/forward.rs:1822-1842.
    """
    logits = np.asarray(logits, dtype=F32)
    if logits.size == 0:
        raise ValueError("cannot select a token from empty logits")
    bad = np.nonzero(~np.isfinite(logits))[0]
    if bad.size:
        raise ValueError(f"logit {int(bad[0])} is not finite: {logits[bad[0]]}")
    return int(np.argmax(logits))


# ----------------------------------------------------------------------------------------
# the model
# ----------------------------------------------------------------------------------------

class PlainConfig:
    """The numbers of config.json that the formulas use."""

    def __init__(self, d):
        self.n_layers = int(d["num_hidden_layers"])
        self.hidden = int(d["hidden_size"])
        self.n_heads = int(d["num_attention_heads"])
        self.n_kv_heads = int(d["num_key_value_heads"])
        self.head_dim = int(d.get("head_dim", self.hidden // self.n_heads))
        self.intermediate = int(d["intermediate_size"])
        self.vocab = int(d["vocab_size"])
        self.eps = float(d["rms_norm_eps"])
        self.theta = float(d["rope_theta"])
        self.tied = bool(d.get("tie_word_embeddings", False))


def load_plain(model_dir):
    """Read config.json and model.safetensors with the safetensors package (not the engine's reader)."""
    from safetensors import safe_open
    import torch

    with open(os.path.join(model_dir, "config.json")) as f:
        cfg = PlainConfig(json.load(f))
    weights = {}
    with safe_open(os.path.join(model_dir, "model.safetensors"), framework="pt") as f:
        for name in f.keys():
            weights[name] = f.get_tensor(name).to(torch.float32).numpy()
    return cfg, weights


def attention_block(cfg, w, prefix, hidden, first_position=0):
    """The attention half of a layer: h + Wo * Attn(...).  Row t stands at position first_position + t
    and sees the rows before it (the reference's chunk at `position_start`, forward.rs:1164-1189, with
    nothing in the cache before it).

    crates/beholdd-model/src/qwen3moe/forward.rs:1075-1252: input RMSNorm; q, k, v
    projections; per-head RMSNorm of q and k with one [head_dim] weight each and the same
    eps, BEFORE the rotation (:1130-1156); split-half rotation of q and k at the absolute
    position (:1161-1189); scale 1/sqrt(head_dim) computed in f32 (:1192); causal GQA
    attention; output projection added to the residual (:1236-1252).
    """
    t_len = hidden.shape[0]
    hd, nh, nkv = cfg.head_dim, cfg.n_heads, cfg.n_kv_heads
    xn = rmsnorm(hidden, w[prefix + "input_layernorm.weight"], cfg.eps)
    q = linear(xn, w[prefix + "self_attn.q_proj.weight"]).reshape(t_len, nh, hd)
    k = linear(xn, w[prefix + "self_attn.k_proj.weight"]).reshape(t_len, nkv, hd)
    v = linear(xn, w[prefix + "self_attn.v_proj.weight"])
    q = rmsnorm(q, w[prefix + "self_attn.q_norm.weight"], cfg.eps)
    k = rmsnorm(k, w[prefix + "self_attn.k_norm.weight"], cfg.eps)
    freqs = rope_frequencies(cfg.theta, hd)
    for t in range(t_len):
        cos, sin = rope_cos_sin(freqs, first_position + t)
        q[t] = rope_split_half(q[t], cos, sin)
        k[t] = rope_split_half(k[t], cos, sin)
    scale = F32(1.0) / np.sqrt(F32(hd))
    attended = causal_attention(q.reshape(t_len, nh * hd), k.reshape(t_len, nkv * hd), v,
                                nh, nkv, hd, scale)
    return (hidden + linear(attended, w[prefix + "self_attn.o_proj.weight"])).astype(F32)


def mlp_block(cfg, w, prefix, hidden):
    """The feed-forward half: h + Wd * (silu(Wg x) * (Wu x)) on the normed input.

    crates/beholdd-model/src/qwen3moe/forward.rs:1256-1298 and :1405-1407.
    """
    xf = rmsnorm(hidden, w[prefix + "post_attention_layernorm.weight"], cfg.eps)
    g = linear(xf, w[prefix + "mlp.gate_proj.weight"])
    u = linear(xf, w[prefix + "mlp.up_proj.weight"])
    out = linear(swiglu(g, u), w[prefix + "mlp.down_proj.weight"])
    return (hidden + out).astype(F32)


def layer(cfg, w, index, hidden, first_position=0):
    """h = h + Attn(RMSNorm(h)); h = h + MLP(RMSNorm(h)).

    crates/beholdd-model/src/qwen3moe/forward.rs:1022-1414.
    """
    prefix = f"model.layers.{index}."
    hidden = attention_block(cfg, w, prefix, hidden, first_position)
    return mlp_block(cfg, w, prefix, hidden)


def head(cfg, w, hidden, rows=None):
    """Final RMSNorm then the LM head (the embedding itself when tied).

    crates/beholdd-model/src/qwen3moe/forward.rs:1416-1455 (there for the last row only;
    here for every row, or for the rows asked for) and crates/beholdd-model/src/qwen3moe.rs:948-955 (tied head).
    """
    if rows is not None:
        hidden = hidden[np.asarray(rows, dtype=np.int64)]
    xl = rmsnorm(hidden, w["model.norm.weight"], cfg.eps)
    out = w["model.embed_tokens.weight"] if cfg.tied else w["lm_head.weight"]
    return linear(xl, out)


def forward_logits(cfg, w, tokens, first_position=0, rows=None):
    """Logits [T, vocab] of every position of one whole sequence (or of the positions `rows`).

    crates/beholdd-model/src/qwen3moe/forward.rs:412-436 (the non-cached forward).
    """
    hidden = embed(tokens, w["model.embed_tokens.weight"])
    for index in range(cfg.n_layers):
        hidden = layer(cfg, w, index, hidden, first_position)
    return head(cfg, w, hidden, rows)


def greedy_generate(cfg, w, prompt, max_new_tokens, stop_tokens=()):
    """Greedy generation by recomputing the whole prefix at every step.

    crates/beholdd-model/src/qwen3moe/forward.rs:597-686: the stop token is selected but
    neither emitted nor appended; the last emitted token is never evaluated.
    Returns (generated, stop_token or None).
    """
    tokens = list(prompt)
    generated = []
    for _ in range(max_new_tokens):
        token = greedy_token(forward_logits(cfg, w, tokens)[-1])
        if token in stop_tokens:
            return generated, token
        generated.append(token)
        tokens.append(token)
    return generated, None
