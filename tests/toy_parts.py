"""Toy parts and toy architectures, defined here and nowhere in the package, to show that a
new mixer with state of its own, a new arrangement of layers and a new architecture can be
registered, built, loaded and stepped without a change to the framework's files.  They are
no model of anyone's."""

from __future__ import annotations

import numpy as np
import torch

import beholdd
import plain_qwen3 as plain
from beholdd.config import LayerKinds, Qwen3Config
from beholdd.models import build_decoder
from beholdd.parts import MIXERS, CacheNeed
from beholdd.weights import TensorSpec

DECAY = 0.75


class ToyRunningMeanMixer:
    """state <- DECAY * state + x_t for every token in order; output = W state.
    Keeps one float32 vector per sequence: a cache need of kind "state".  A step of one token per sequence
    uses the step's device tensors only, so decode steps of a model with this mixer may be captured and
    replayed; steps of several tokens are never captured and scan on the host."""

    graph_safe = True

    def __init__(self, hidden: int, prefix: str):
        self.hidden, self.name = hidden, prefix + "toy_mix.weight"
        self.weight = None

    def tensor_specs(self):
        return [TensorSpec(self.name, (self.hidden, self.hidden), "linear")]

    def load(self, get):
        self.weight = get(self.name)

    def cache_need(self):
        return CacheNeed(kind="state", state_shape=(self.hidden,), state_dtype=torch.float32)

    def forward(self, ctx, x, hidden, cache):
        if ctx.is_decode:
            slots = ctx.seq_slot.long()
            state = cache.state.index_select(0, slots) * DECAY + x.float()
            cache.state.index_copy_(0, slots, state)
            ctx.kernels.gemm(state, self.weight, hidden, accumulate=True)
            return
        for b in range(ctx.n_seqs):
            lo, hi = ctx.host_seq_start[b], ctx.host_seq_start[b + 1]
            state = cache.state[ctx.host_seq_slot[b]]
            for row in range(lo, hi):          # a scan: rows of one sequence in order
                state.mul_(DECAY).add_(x[row].float())
                hidden[row] += (self.weight.float() @ state)


def plain_toy_mixer(xn, weight):
    state = np.zeros(xn.shape[1], np.float32)
    out = np.zeros_like(xn)
    for t in range(xn.shape[0]):
        state = (np.float32(DECAY) * state + xn[t]).astype(np.float32)
        out[t] = (weight.astype(np.float64) @ state.astype(np.float64)).astype(np.float32)
    return out


class ToyHybridConfig(Qwen3Config):
    """Attention in even layers, the toy mixer in odd ones."""

    def layer_kinds(self):
        return [LayerKinds(mixer="gqa_attention" if i % 2 == 0 else "toy_running_mean", feed_forward="swiglu",
                           norm="rmsnorm", block="pre_norm") for i in range(self.n_layers)]


class ToyTwiceConfig(Qwen3Config):
    """Layer 0 runs again after the last layer, with a cache entry of its own."""

    def schedule(self):
        return [(i, i) for i in range(self.n_layers)] + [(0, self.n_layers)]


class ToySharedCacheConfig(Qwen3Config):
    """Every odd layer reads the keys and values that the layer before it wrote."""

    def schedule(self):
        return [(i, i - (i % 2)) for i in range(self.n_layers)]


def register():
    if "toy_running_mean" not in MIXERS:
        MIXERS.register("toy_running_mean", lambda config, index, prefix, shared: ToyRunningMeanMixer(config.hidden, prefix))
    for name, cls in (("ToyHybridForCausalLM", ToyHybridConfig), ("ToyTwiceForCausalLM", ToyTwiceConfig),
                      ("ToySharedCacheForCausalLM", ToySharedCacheConfig)):
        if name not in beholdd.registered_architectures():
            beholdd.register_architecture(name, cls, build_decoder)


def unregister():
    MIXERS.unregister("toy_running_mean")
    for name in ("ToyHybridForCausalLM", "ToyTwiceForCausalLM", "ToySharedCacheForCausalLM"):
        beholdd.registry.unregister_architecture(name)


BASE = {
    "num_hidden_layers": 4, "hidden_size": 48, "num_attention_heads": 3, "num_key_value_heads": 1, "head_dim": 16,
    "intermediate_size": 80, "vocab_size": 101, "rope_theta": 10000.0, "rms_norm_eps": 1e-5,
    "max_position_embeddings": 512, "tie_word_embeddings": False,
}


def config_dict(architecture):
    return dict(BASE, architectures=[architecture])


# ---- plain forms of the toy architectures --------------------------------------------------------

def _attention_parts(cfg, w, prefix, hidden):
    """q, k, v of one layer (normed, rotated), for all positions."""
    t_len, hd = hidden.shape[0], cfg.head_dim
    xn = plain.rmsnorm(hidden, w[prefix + "input_layernorm.weight"], cfg.eps)
    q = plain.rmsnorm(plain.linear(xn, w[prefix + "self_attn.q_proj.weight"]).reshape(t_len, cfg.n_heads, hd),
                      w[prefix + "self_attn.q_norm.weight"], cfg.eps)
    k = plain.rmsnorm(plain.linear(xn, w[prefix + "self_attn.k_proj.weight"]).reshape(t_len, cfg.n_kv_heads, hd),
                      w[prefix + "self_attn.k_norm.weight"], cfg.eps)
    v = plain.linear(xn, w[prefix + "self_attn.v_proj.weight"])
    freqs = plain.rope_frequencies(cfg.theta, hd)
    for t in range(t_len):
        cs = plain.rope_cos_sin(freqs, t)
        q[t], k[t] = plain.rope_split_half(q[t], *cs), plain.rope_split_half(k[t], *cs)
    return q.reshape(t_len, -1), k.reshape(t_len, -1), v


def plain_logits(architecture, cfg, w, tokens):
    hidden = plain.embed(tokens, w["model.embed_tokens.weight"])
    scale = np.float32(1) / np.sqrt(np.float32(cfg.head_dim))
    if architecture == "ToyHybridForCausalLM":
        for i in range(cfg.n_layers):
            prefix = f"model.layers.{i}."
            if i % 2 == 0:
                hidden = plain.attention_block(cfg, w, prefix, hidden)
            else:
                xn = plain.rmsnorm(hidden, w[prefix + "input_layernorm.weight"], cfg.eps)
                hidden = (hidden + plain_toy_mixer(xn, w[prefix + "toy_mix.weight"])).astype(np.float32)
            hidden = plain.mlp_block(cfg, w, prefix, hidden)
    elif architecture == "ToyTwiceForCausalLM":
        for i in list(range(cfg.n_layers)) + [0]:
            hidden = plain.layer(cfg, w, i, hidden)
    elif architecture == "ToySharedCacheForCausalLM":
        shared = None
        for i in range(cfg.n_layers):
            prefix = f"model.layers.{i}."
            q, k, v = _attention_parts(cfg, w, prefix, hidden)
            if i % 2 == 0:
                shared = (k, v)
            attended = plain.causal_attention(q, shared[0], shared[1], cfg.n_heads, cfg.n_kv_heads, cfg.head_dim, scale)
            hidden = (hidden + plain.linear(attended, w[prefix + "self_attn.o_proj.weight"])).astype(np.float32)
            hidden = plain.mlp_block(cfg, w, prefix, hidden)
    else:
        raise ValueError(architecture)
    return plain.head(cfg, w, hidden)


def check_architecture(architecture, folder, make_engine, tolerance):
    """Whole, one by one and in batches: all equal to the plain form."""
    import schedules

    cfg, weights = plain.load_plain(folder)
    requests = schedules.random_requests(cfg.vocab, [3, 70, 21, 40], seed=13)
    want = [plain_logits(architecture, cfg, weights, r) for r in requests]
    engine = make_engine(folder)
    for label, got in (("whole", schedules.whole(engine, requests)),
                       ("one by one", schedules.tail_one_by_one(engine, requests, tail=32)),
                       ("batches", schedules.batches(engine, requests, batch_size=3))):
        for index, (g, e) in enumerate(zip(got, want)):
            error = schedules.relative_error(g, e)
            assert error < tolerance, (architecture, label, index, error)
    engine.cache.check_invariants()
    return engine
