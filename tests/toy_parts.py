"""Toy parts and toy architectures, defined here and nowhere in the package, to show that a
new mixer with state of its own, a new arrangement of layers and a new architecture can be
registered, built, loaded and stepped without a change to the framework's files.  They are
no model of anyone's."""

from __future__ import annotations

import numpy as np
import torch

import beholdd
import plain_qwen3 as plain
from dataclasses import dataclass

from beholdd.config import ConfigReader, LayerKinds, Qwen3Config
from beholdd.models import build_decoder
from beholdd.parts import (BLOCKS, FEED_FORWARDS, MIXERS, NORMS, POSITION_ENCODINGS, CacheNeed, GQAAttention, Linear, RMSNorm,
                           RotaryEncoding, SwiGLU)
from beholdd.parts.embedding import Embedding, LMHead
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


# ---- a norm and an arrangement of a layer's parts of another make ----------------------------------------

class ToyCentredNorm:
    """y = (x - mean) / sqrt(mean((x - mean)^2) + eps) * weight + bias, the statistics in float32 on the float32
    residual: two tensors and a mean where the package's norm has one tensor and none.  Device tensors only, for
    steps of any shape."""

    graph_safe = True
    graph_safe_rows = None

    def __init__(self, width: int, eps: float, name: str):
        self.width, self.eps, self.name, self.bias_name = width, eps, name, name.replace(".weight", ".bias")
        self.weight = self.bias = None

    def tensor_specs(self):
        return [TensorSpec(self.name, (self.width,), "norm"), TensorSpec(self.bias_name, (self.width,), "linear")]

    def load(self, get):
        self.weight, self.bias = get(self.name), get(self.bias_name)

    def forward(self, ctx, hidden, rows=None):
        x = hidden if rows is None else hidden.index_select(0, rows.long())
        centred = x - x.mean(dim=-1, keepdim=True)
        y = centred * torch.rsqrt(centred.pow(2).mean(dim=-1, keepdim=True) + self.eps) * self.weight.float() + self.bias.float()
        return y.to(ctx.act_dtype)


def plain_centred_norm(x, weight, bias, eps):
    x = x.astype(np.float32)
    centred = x - x.mean(axis=-1, keepdims=True, dtype=np.float32)
    inv = np.float32(1) / np.sqrt((centred * centred).mean(axis=-1, keepdims=True, dtype=np.float32) + np.float32(eps))
    return (centred * inv * weight.astype(np.float32) + bias.astype(np.float32)).astype(np.float32)


class ToyParallelBlock:
    """h = h + Mixer(Norm(h)) + FeedForward(Norm(h)): one norm, and the mixer and the feed-forward both read what it
    wrote of the layer's input (the package's block norms twice and feeds the second norm what the mixer added)."""

    def __init__(self, norm, mixer, feed_forward):
        self.norm, self.mixer, self.feed_forward = norm, mixer, feed_forward

    def parts(self):
        return [self.norm, self.mixer, self.feed_forward]

    @property
    def graph_safe(self):
        return all(getattr(part, "graph_safe", False) for part in self.parts())

    @property
    def graph_safe_rows(self):
        from beholdd.parts.base import graph_rows_allowed
        return graph_rows_allowed(self.parts())

    def tensor_specs(self):
        return [spec for part in self.parts() for spec in part.tensor_specs()]

    def load(self, get):
        for part in self.parts():
            part.load(get)

    def prepare(self, kernels):
        for part in self.parts():
            if hasattr(part, "prepare"):
                part.prepare(kernels)

    def cache_need(self):
        return self.mixer.cache_need()

    def forward(self, ctx, hidden, cache, prepared=None, next_block=None):
        x = self.norm.forward(ctx, hidden)
        self.mixer.forward(ctx, x, hidden, cache)
        self.feed_forward.forward(ctx, x, hidden)
        return None


class ToyScaledEmbedding(Embedding):
    """The embedding's rows times sqrt(width), in float32."""

    def forward(self, ctx):
        return super().forward(ctx).mul_(float(np.sqrt(np.float32(self.width))))


LOGIT_CAP = 0.5


class ToyCappedHead(LMHead):
    """Logits held within (-LOGIT_CAP, LOGIT_CAP): cap * tanh(logits / cap), in float32."""

    def forward(self, ctx, x):
        logits = super().forward(ctx, x)
        return torch.tanh(logits / LOGIT_CAP) * LOGIT_CAP


def build_toy_parallel_model(config):
    return build_decoder(config, make_embedding=lambda c: ToyScaledEmbedding(c.vocab, c.hidden, "model.embed_tokens.weight"),
                         make_head=lambda c, embedding: ToyCappedHead(c.vocab, c.hidden, "lm_head.weight"))


class ToyParallelConfig(Qwen3Config):
    """Odd layers in the parallel arrangement with the centred norm, even ones as the package has them."""

    def layer_kinds(self):
        return [LayerKinds(mixer="gqa_attention", feed_forward="swiglu", norm="toy_centred_norm" if i % 2 else "rmsnorm",
                           block="toy_parallel" if i % 2 else "pre_norm") for i in range(self.n_layers)]


def _build_toy_parallel(config, layer_index, prefix, kinds, shared):
    return ToyParallelBlock(NORMS.get(kinds.norm)(config, config.hidden, prefix + "input_layernorm.weight", shared),
                            MIXERS.get(kinds.mixer)(config, layer_index, prefix, shared),
                            FEED_FORWARDS.get(kinds.feed_forward)(config, layer_index, prefix, shared))


# ---- attention over a window of the keys in some layers, over all of them in the others ---------------------

WINDOW = 24


class ToyWindowedConfig(Qwen3Config):
    """Odd layers see the last WINDOW keys only: their keys and values get storage of their own, which gives
    pages back as a sequence moves on; even layers see all keys."""

    def layer_kinds(self):
        return [LayerKinds(mixer="toy_windowed_attention" if i % 2 else "gqa_attention", feed_forward="swiglu",
                           norm="rmsnorm", block="pre_norm") for i in range(self.n_layers)]


def plain_windowed_attention(q, k, v, n_heads, n_kv_heads, head_dim, scale, window):
    """Query t sees keys max(0, t - window + 1) .. t: scores in float32 from float64 dot products, softmax in float32."""
    t_len = q.shape[0]
    qh, kh, vh = (a.astype(np.float64).reshape(t_len, -1, head_dim) for a in (q, k, v))
    out = np.zeros((t_len, n_heads, head_dim), np.float32)
    for h in range(n_heads):
        g = h // (n_heads // n_kv_heads)
        for t in range(t_len):
            lo = max(0, t - window + 1)
            scores = ((kh[lo:t + 1, g] @ qh[t, h]) * np.float64(np.float32(scale))).astype(np.float32)
            out[t, h] = (plain.softmax(scores).astype(np.float64) @ vh[lo:t + 1, g]).astype(np.float32)
    return out.reshape(t_len, -1)


# ---- an architecture with a configuration of its own ----------------------------------------------------
# Its config.json has other keys, its configuration class inherits nothing from Qwen3's, its tensors have
# other names, and it brings a feed-forward with routing and a position encoding of its own; the builders
# below adapt its fields to the parts' constructor parameters.

class ToyRoutedFeedForward:
    """Top-1 routing over a few small SwiGLU experts: router logits and their softmax in float32; each row goes
    to its most likely expert (ties to the lowest index), whose output is scaled by that probability.
    Keeps the last step's routing for inspection."""

    def __init__(self, hidden: int, width: int, n_experts: int, prefix: str):
        self.hidden, self.width, self.n_experts = hidden, width, n_experts
        self.router = Linear(hidden, n_experts, prefix + "router.weight")
        self.experts = [SwiGLU(hidden, width, f"{prefix}experts.{e}.") for e in range(n_experts)]
        self.last_routing = None

    def tensor_specs(self):
        return self.router.tensor_specs() + [spec for expert in self.experts for spec in expert.tensor_specs()]

    def load(self, get):
        self.router.load(get)
        for expert in self.experts:
            expert.load(get)

    def forward(self, ctx, x, hidden):
        logits = self.router.forward(ctx, x, out_dtype=torch.float32)
        probabilities = torch.softmax(logits, dim=-1)
        chosen = probabilities.argmax(dim=-1)
        self.last_routing = chosen
        ctx.extras.setdefault("routing", {})[self.router.names[0]] = chosen       # the step's second way out
        for index, expert in enumerate(self.experts):
            rows = torch.nonzero(chosen == index).flatten()
            if rows.numel() == 0:
                continue
            out = torch.zeros((rows.numel(), self.hidden), dtype=torch.float32, device=hidden.device)
            expert.forward(ctx, x.index_select(0, rows).contiguous(), out)
            hidden.index_add_(0, rows, out * probabilities[rows, index].unsqueeze(1))


class ToyStretchedRotary(RotaryEncoding):
    """Rotates only the first `rotary_dim` dimensions of a head, at position / stretch."""

    def __init__(self, rotary_dim, theta, max_position, stretch):
        super().__init__(rotary_dim, theta, max_position)
        self.stretch = float(stretch)

    def build_tables(self, device):
        half = self.rotary_dim // 2
        freqs = np.array([1.0 / (self.theta ** ((2 * i) / self.rotary_dim)) for i in range(half)], dtype=np.float64)
        angles = (np.arange(self.max_position, dtype=np.float64) / self.stretch)[:, None] * freqs[None, :]
        self._tables = (torch.from_numpy(np.cos(angles).astype(np.float32)).to(device).contiguous(),
                        torch.from_numpy(np.sin(angles).astype(np.float32)).to(device).contiguous())


@dataclass(frozen=True)
class ToyOwnConfig:
    depth: int
    width: int
    readers: int            # query heads
    stores: int             # key/value heads
    head_size: int
    turned: int             # dimensions of a head that the position encoding rotates
    stretch: float
    base: float
    inner: int              # feed-forward width
    experts: int
    symbols: int
    floor: float            # the norms' epsilon
    longest: int

    @classmethod
    def from_dict(cls, data, origin="config.json"):
        r = ConfigReader(data, origin)
        return cls(depth=r.integer("toy_depth", minimum=1), width=r.integer("toy_width", minimum=1),
                   readers=r.integer("toy_readers", minimum=1), stores=r.integer("toy_stores", minimum=1),
                   head_size=r.integer("toy_head_size", minimum=2), turned=r.integer("toy_turned", minimum=2),
                   stretch=r.number("toy_stretch"), base=r.number("toy_base"), inner=r.integer("toy_inner", minimum=1),
                   experts=r.integer("toy_experts", minimum=1), symbols=r.integer("toy_symbols", minimum=1),
                   floor=r.number("toy_floor"), longest=r.integer("toy_longest", minimum=1))

    # what the generic builder reads
    vocab = property(lambda self: self.symbols)
    hidden = property(lambda self: self.width)
    max_position = property(lambda self: self.longest)
    tie_word_embeddings = False

    def layer_kinds(self):
        """Attention and a routed feed-forward in even layers, the state mixer and a dense one in odd layers."""
        return [LayerKinds(mixer="toy_own_attention" if i % 2 == 0 else "toy_own_running_mean",
                           feed_forward="toy_routed" if i % 2 == 0 else "toy_own_swiglu",
                           norm="toy_own_rmsnorm", block="pre_norm") for i in range(self.depth)]

    def schedule(self):
        return [(i, i) for i in range(self.depth)]


def build_toy_own(config):
    return build_decoder(config, position_encoding={"early": "toy_stretched_rotary", "late": "none"}, layer_prefix="blocks.{}.",
                         embedding_name="symbols.weight", final_norm_name="last_norm.weight",
                         head_name="readout.weight", final_norm_kind="toy_own_rmsnorm")


OWN_PARTS = (
    (MIXERS, "toy_own_attention", lambda c, index, prefix, shared: GQAAttention(
        c.width, c.readers, c.stores, c.head_size, prefix + "look.", qk_norm_eps=c.floor,
        position_encoding=shared["position_encodings"]["early" if index < c.depth // 2 else "late"])),
    (MIXERS, "toy_own_running_mean", lambda c, index, prefix, shared: ToyRunningMeanMixer(c.width, prefix)),
    (FEED_FORWARDS, "toy_routed", lambda c, index, prefix, shared: ToyRoutedFeedForward(c.width, c.inner, c.experts, prefix + "routed.")),
    (FEED_FORWARDS, "toy_own_swiglu", lambda c, index, prefix, shared: SwiGLU(c.width, c.inner, prefix + "dense.")),
    (NORMS, "toy_own_rmsnorm", lambda c, width, name, shared: RMSNorm(width, c.floor, name)),
    (POSITION_ENCODINGS, "toy_stretched_rotary", lambda c, shared: ToyStretchedRotary(c.turned, c.base, c.longest, c.stretch)),
    (NORMS, "toy_centred_norm", lambda c, width, name, shared: ToyCentredNorm(width, c.rms_eps, name)),
    (MIXERS, "toy_windowed_attention", lambda c, index, prefix, shared: GQAAttention(
        c.hidden, c.n_heads, c.n_kv_heads, c.head_dim, prefix + "self_attn.", position_encoding=shared["position_encoding"],
        qk_norm_eps=c.rms_eps, window=WINDOW)),
    (BLOCKS, "toy_parallel", _build_toy_parallel),
)

OWN = {
    "architectures": ["ToyOwnForCausalLM"], "toy_depth": 4, "toy_width": 40, "toy_readers": 4, "toy_stores": 2,
    "toy_head_size": 24, "toy_turned": 16, "toy_stretch": 2.5, "toy_base": 500.0, "toy_inner": 56, "toy_experts": 3,
    "toy_symbols": 90, "toy_floor": 1e-5, "toy_longest": 512,
}


def register():
    if "toy_running_mean" not in MIXERS:
        MIXERS.register("toy_running_mean", lambda config, index, prefix, shared: ToyRunningMeanMixer(config.hidden, prefix))
    for registry, name, builder in OWN_PARTS:
        if name not in registry:
            registry.register(name, builder)
    for name, cls, build in (("ToyHybridForCausalLM", ToyHybridConfig, build_decoder),
                             ("ToyTwiceForCausalLM", ToyTwiceConfig, build_decoder),
                             ("ToySharedCacheForCausalLM", ToySharedCacheConfig, build_decoder),
                             ("ToyParallelForCausalLM", ToyParallelConfig, build_toy_parallel_model),
                             ("ToyWindowedForCausalLM", ToyWindowedConfig, build_decoder),
                             ("ToyOwnForCausalLM", ToyOwnConfig, build_toy_own)):
        if name not in beholdd.registered_architectures():
            beholdd.register_architecture(name, cls, build)


def unregister():
    MIXERS.unregister("toy_running_mean")
    for registry, name, _ in OWN_PARTS:
        registry.unregister(name)
    for name in ("ToyHybridForCausalLM", "ToyTwiceForCausalLM", "ToySharedCacheForCausalLM", "ToyParallelForCausalLM",
                 "ToyWindowedForCausalLM", "ToyOwnForCausalLM"):
        beholdd.registry.unregister_architecture(name)


BASE = {
    "num_hidden_layers": 4, "hidden_size": 48, "num_attention_heads": 3, "num_key_value_heads": 1, "head_dim": 16,
    "intermediate_size": 80, "vocab_size": 101, "rope_theta": 10000.0, "rms_norm_eps": 1e-5,
    "max_position_embeddings": 512, "tie_word_embeddings": False,
}


def config_dict(architecture):
    if architecture == "ToyOwnForCausalLM":
        return dict(OWN)
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


def plain_own_logits(config, w, tokens):
    """The plain form of ToyOwnForCausalLM from the plain implementation's part functions."""
    c = ToyOwnConfig.from_dict(config)
    hidden = plain.embed(tokens, w["symbols.weight"])
    t_len, hd = hidden.shape[0], c.head_size
    freqs = plain.rope_frequencies(c.base, c.turned)
    scale = np.float32(1) / np.sqrt(np.float32(hd))
    routing = []
    for i in range(c.depth):
        p = f"blocks.{i}."
        xn = plain.rmsnorm(hidden, w[p + "input_layernorm.weight"], c.floor)
        if i % 2 == 0:
            q = plain.rmsnorm(plain.linear(xn, w[p + "look.q_proj.weight"]).reshape(t_len, c.readers, hd), w[p + "look.q_norm.weight"], c.floor)
            k = plain.rmsnorm(plain.linear(xn, w[p + "look.k_proj.weight"]).reshape(t_len, c.stores, hd), w[p + "look.k_norm.weight"], c.floor)
            v = plain.linear(xn, w[p + "look.v_proj.weight"])
            for t in range(t_len if i < c.depth // 2 else 0):      # the later layers' attention has no position encoding
                cs = plain.rope_cos_sin(freqs, t / c.stretch)
                q[t, :, :c.turned] = plain.rope_split_half(q[t, :, :c.turned], *cs)
                k[t, :, :c.turned] = plain.rope_split_half(k[t, :, :c.turned], *cs)
            attended = plain.causal_attention(q.reshape(t_len, -1), k.reshape(t_len, -1), v, c.readers, c.stores, hd, scale)
            hidden = (hidden + plain.linear(attended, w[p + "look.o_proj.weight"])).astype(np.float32)
        else:
            hidden = (hidden + plain_toy_mixer(xn, w[p + "toy_mix.weight"])).astype(np.float32)
        xf = plain.rmsnorm(hidden, w[p + "post_attention_layernorm.weight"], c.floor)
        if i % 2 == 0:
            probabilities = plain.softmax(plain.linear(xf, w[p + "routed.router.weight"]))
            chosen = probabilities.argmax(axis=-1)
            routing.append(chosen)
            out = np.zeros_like(hidden)
            for t in range(t_len):
                e = f"{p}routed.experts.{chosen[t]}."
                a = plain.swiglu(plain.linear(xf[t], w[e + "gate_proj.weight"]), plain.linear(xf[t], w[e + "up_proj.weight"]))
                out[t] = plain.linear(a, w[e + "down_proj.weight"]) * probabilities[t, chosen[t]]
            hidden = (hidden + out).astype(np.float32)
        else:
            a = plain.swiglu(plain.linear(xf, w[p + "dense.gate_proj.weight"]), plain.linear(xf, w[p + "dense.up_proj.weight"]))
            hidden = (hidden + plain.linear(a, w[p + "dense.down_proj.weight"])).astype(np.float32)
    return plain.linear(plain.rmsnorm(hidden, w["last_norm.weight"], c.floor), w["readout.weight"]), routing


def load_plain_weights(folder):
    """(config.json as a dictionary, tensors as float32 arrays) of any model folder."""
    import json
    import os
    from safetensors import safe_open

    with open(os.path.join(folder, "config.json")) as handle:
        config = json.load(handle)
    with safe_open(os.path.join(folder, "model.safetensors"), framework="pt") as handle:
        return config, {name: handle.get_tensor(name).to(torch.float32).numpy() for name in handle.keys()}


def plain_logits(architecture, cfg, w, tokens):
    if architecture == "ToyOwnForCausalLM":
        return plain_own_logits(cfg, w, tokens)[0]
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
    elif architecture == "ToyWindowedForCausalLM":
        for i in range(cfg.n_layers):
            prefix = f"model.layers.{i}."
            if i % 2:
                q, k, v = _attention_parts(cfg, w, prefix, hidden)
                attended = plain_windowed_attention(q, k, v, cfg.n_heads, cfg.n_kv_heads, cfg.head_dim, scale, WINDOW)
                hidden = (hidden + plain.linear(attended, w[prefix + "self_attn.o_proj.weight"])).astype(np.float32)
            else:
                hidden = plain.attention_block(cfg, w, prefix, hidden)
            hidden = plain.mlp_block(cfg, w, prefix, hidden)
    elif architecture == "ToyParallelForCausalLM":
        hidden = (hidden * np.sqrt(np.float32(cfg.hidden))).astype(np.float32)      # the scaled embedding
        freqs = plain.rope_frequencies(cfg.theta, cfg.head_dim)
        for i in range(cfg.n_layers):
            prefix = f"model.layers.{i}."
            if i % 2 == 0:
                hidden = plain.layer(cfg, w, i, hidden)
                continue
            t_len, hd = hidden.shape[0], cfg.head_dim
            xn = plain_centred_norm(hidden, w[prefix + "input_layernorm.weight"], w[prefix + "input_layernorm.bias"], cfg.eps)
            q = plain.rmsnorm(plain.linear(xn, w[prefix + "self_attn.q_proj.weight"]).reshape(t_len, cfg.n_heads, hd),
                              w[prefix + "self_attn.q_norm.weight"], cfg.eps)
            k = plain.rmsnorm(plain.linear(xn, w[prefix + "self_attn.k_proj.weight"]).reshape(t_len, cfg.n_kv_heads, hd),
                              w[prefix + "self_attn.k_norm.weight"], cfg.eps)
            v = plain.linear(xn, w[prefix + "self_attn.v_proj.weight"])
            for t in range(t_len):
                cs = plain.rope_cos_sin(freqs, t)
                q[t], k[t] = plain.rope_split_half(q[t], *cs), plain.rope_split_half(k[t], *cs)
            attended = plain.causal_attention(q.reshape(t_len, -1), k.reshape(t_len, -1), v, cfg.n_heads, cfg.n_kv_heads, hd, scale)
            mixed = plain.linear(attended, w[prefix + "self_attn.o_proj.weight"])
            fed = plain.linear(plain.swiglu(plain.linear(xn, w[prefix + "mlp.gate_proj.weight"]), plain.linear(xn, w[prefix + "mlp.up_proj.weight"])),
                               w[prefix + "mlp.down_proj.weight"])
            hidden = ((hidden + mixed).astype(np.float32) + fed).astype(np.float32)      # the engine adds the two in this order
        logits = plain.head(cfg, w, hidden).astype(np.float32)
        return (np.tanh(logits / np.float32(LOGIT_CAP)) * np.float32(LOGIT_CAP)).astype(np.float32)      # the capped head
    else:
        raise ValueError(architecture)
    return plain.head(cfg, w, hidden)


def check_architecture(architecture, folder, make_engine, tolerance):
    """Whole, one by one and in batches: all equal to the plain form."""
    import schedules

    if architecture == "ToyOwnForCausalLM":
        cfg, weights = load_plain_weights(folder)
        vocab = cfg["toy_symbols"]
    else:
        cfg, weights = plain.load_plain(folder)
        vocab = cfg.vocab
    # (with a window, one request long enough for the windowed layers to give pages back while it is decoded)
    requests = schedules.random_requests(vocab, [3, 70, 21, 40] + ([150] if architecture == "ToyWindowedForCausalLM" else []), seed=13)
    want = [plain_logits(architecture, cfg, weights, r) for r in requests]
    engine = make_engine(folder)
    for label, got in (("whole", schedules.whole(engine, requests)),
                       ("one by one", schedules.tail_one_by_one(engine, requests, tail=32)),
                       ("batches", schedules.batches(engine, requests, batch_size=3)),
                       ("portions", schedules.portions(engine, requests))):
        for index, (g, e) in enumerate(zip(got, want)):
            error = schedules.relative_error(g, e)
            assert error < tolerance, (architecture, label, index, error)
    engine.cache.check_invariants()
    return engine
