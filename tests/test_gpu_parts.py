"""Each part alone on the GPU against the plain function of the same formula, and the toy
parts and architectures of tests/toy_parts.py through the real kernels."""

import math

import numpy as np
import pytest
import torch

import beholdd
import plain_qwen3 as plain
import schedules
import toy_parts
from beholdd.cache import SequenceCache
from beholdd.engine import Engine, StepEntry, build_step
from beholdd.parts import (Embedding, GQAAttention, LMHead, Linear, NoPositionEncoding, PreNormBlock, RMSNorm,
                           RotaryEncoding, SwiGLU)

pytestmark = pytest.mark.gpu
DEVICE = "cuda:0"
DTYPES = [torch.float32, torch.bfloat16]


@pytest.fixture(scope="module")
def K():
    from beholdd.kernels import HipKernels
    return HipKernels(DEVICE)


class Weights:
    """Random tensors for a part's specs; hands them out on the device in the part's dtype."""

    def __init__(self, specs, dtype, seed=0, std=0.08):
        g = torch.Generator().manual_seed(seed)
        self.host = {}
        for spec in specs:
            value = torch.randn(spec.shape, generator=g) * std + (1.0 if spec.init == "norm" else 0.0)
            self.host[spec.name] = value.to(dtype)
        self.numpy = {name: value.float().numpy() for name, value in self.host.items()}

    def __call__(self, name):
        return self.host[name].to(DEVICE)


def make_ctx(K, dtype, entry_needs, entries, vocab=1000, max_tokens=1024, cache=None):
    if cache is None:
        cache = SequenceCache(entry_needs, max_tokens, dtype, DEVICE, K.page_size)
        cache.allocate()
    built = []
    for tokens in entries:
        built.append(StepEntry(cache.alloc_slot(), list(tokens), []))
    requests = [(entry.slot, len(entry.tokens)) for entry in built]
    cache.reserve(requests)
    ctx, _, tables = build_step(K, dtype, DEVICE, cache, built)
    return ctx, cache, tables, requests


def rel(got, want):
    return schedules.relative_error(got.float().cpu().numpy(), want)


def tol(dtype):
    return 2e-5 if dtype == torch.float32 else 1.2e-2


@pytest.mark.parametrize("dtype", DTYPES)
def test_rmsnorm_part(K, dtype):
    part = RMSNorm(200, 1e-5, "n.weight")
    w = Weights(part.tensor_specs(), dtype)
    part.load(w)
    ctx, *_ = make_ctx(K, dtype, {}, [[1, 2, 3], [4]])
    hidden = torch.randn(4, 200) * 2 + 1
    out = part.forward(ctx, hidden.to(DEVICE))
    assert out.dtype == dtype
    assert rel(out, plain.rmsnorm(hidden.numpy(), w.numpy["n.weight"], 1e-5)) < tol(dtype)
    rows = torch.tensor([3, 0], dtype=torch.int32, device=DEVICE)
    assert rel(part.forward(ctx, hidden.to(DEVICE), rows=rows),
               plain.rmsnorm(hidden.numpy()[[3, 0]], w.numpy["n.weight"], 1e-5)) < tol(dtype)


@pytest.mark.parametrize("dtype", DTYPES)
def test_linear_stacks_tensors_row_by_row(K, dtype):
    part = Linear(72, [40, 24], ["a.weight", "b.weight"])
    w = Weights(part.tensor_specs(), dtype)
    part.load(w)
    ctx, *_ = make_ctx(K, dtype, {}, [[1, 2, 3, 4, 5]])
    x = torch.randn(5, 72).to(dtype)
    out = part.forward(ctx, x.to(DEVICE))
    want = np.concatenate([plain.linear(x.float().numpy(), w.numpy["a.weight"]),
                           plain.linear(x.float().numpy(), w.numpy["b.weight"])], axis=1)
    assert out.shape == (5, 64) and rel(out, want) < tol(dtype)


@pytest.mark.parametrize("dtype", DTYPES)
def test_swiglu_part_adds_into_the_residual(K, dtype):
    part = SwiGLU(96, 200, "mlp.")
    w = Weights(part.tensor_specs(), dtype)
    part.load(w)
    ctx, *_ = make_ctx(K, dtype, {}, [[1] * 7])
    x = torch.randn(7, 96).to(dtype)
    hidden = torch.randn(7, 96)
    residual = hidden.clone().to(DEVICE)
    part.forward(ctx, x.to(DEVICE), residual)
    xn = x.float().numpy()
    inner = plain.swiglu(plain.linear(xn, w.numpy["mlp.gate_proj.weight"]), plain.linear(xn, w.numpy["mlp.up_proj.weight"]))
    want = hidden.numpy() + plain.linear(inner, w.numpy["mlp.down_proj.weight"])
    assert residual.dtype == torch.float32 and rel(residual, want) < tol(dtype)


@pytest.mark.parametrize("dtype", DTYPES)
def test_embedding_and_heads(K, dtype):
    embedding = Embedding(331, 48, "e.weight")
    w = Weights(embedding.tensor_specs(), dtype)
    embedding.load(w)
    ctx, *_ = make_ctx(K, dtype, {}, [[330, 0, 7], [12]], vocab=331)
    hidden = embedding.forward(ctx)
    assert hidden.dtype == torch.float32
    assert np.array_equal(hidden.cpu().numpy(), plain.embed([330, 0, 7, 12], w.numpy["e.weight"]))
    tied = LMHead(331, 48, None, tied_to=embedding)
    tied.load(w)
    assert tied.tensor_specs() == [] and tied.linear.weight.data_ptr() == embedding.weight.data_ptr()
    x = torch.randn(2, 48).to(dtype)
    logits = tied.forward(ctx, x.to(DEVICE))
    assert logits.dtype == torch.float32 and rel(logits, plain.linear(x.float().numpy(), w.numpy["e.weight"])) < tol(dtype)
    own = LMHead(331, 48, "head.weight")
    assert [s.name for s in own.tensor_specs()] == ["head.weight"]


def plain_attention_part(x, w, n_heads, kv_heads, head_dim, eps, theta, scale, window, pasts, news):
    """The attention mixer's formula from the plain functions, for ragged sequences that are
    laid out row after row; sequence s has `pasts[s]` earlier tokens (their rows come first)."""
    outs, at = [], 0
    for n in [p + m for p, m in zip(pasts, news)]:
        xs = x[at:at + n]
        q = plain.linear(xs, w["a.q_proj.weight"]).reshape(n, n_heads, head_dim)
        k = plain.linear(xs, w["a.k_proj.weight"]).reshape(n, kv_heads, head_dim)
        v = plain.linear(xs, w["a.v_proj.weight"])
        if eps is not None:
            q, k = plain.rmsnorm(q, w["a.q_norm.weight"], eps), plain.rmsnorm(k, w["a.k_norm.weight"], eps)
        if theta is not None:
            freqs = plain.rope_frequencies(theta, head_dim)
            for t in range(n):
                cs = plain.rope_cos_sin(freqs, t)
                q[t], k[t] = plain.rope_split_half(q[t], *cs), plain.rope_split_half(k[t], *cs)
        q, k = q.reshape(n, -1), k.reshape(n, -1)
        if window:
            rows = []
            for t in range(n):
                first = max(0, t - window + 1)
                rows.append(plain.causal_attention(q[t:t + 1], k[first:t + 1], v[first:t + 1], n_heads, kv_heads,
                                                   head_dim, scale, query_start=t - first))
            attended = np.concatenate(rows)
        else:
            attended = plain.causal_attention(q, k, v, n_heads, kv_heads, head_dim, scale)
        outs.append(plain.linear(attended, w["a.o_proj.weight"]))
        at += n
    return outs


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("n_heads,kv_heads,head_dim,eps,theta,window", [
    (4, 2, 16, 1e-6, 10000.0, 0),        # the Qwen3 form
    (6, 2, 48, None, None, 0),           # plain attention: no norm, no rotation
    (1, 1, 32, 1e-5, 500.0, 0),          # one head
    (8, 2, 128, 1e-6, 1000000.0, 0),
    (4, 1, 64, 1e-6, 10000.0, 70),       # a window
])
def test_attention_part_in_two_steps(K, dtype, n_heads, kv_heads, head_dim, eps, theta, window):
    hidden_size = 88
    rope = RotaryEncoding(head_dim, theta, 512) if theta is not None else NoPositionEncoding()
    rope.build_tables(DEVICE)
    part = GQAAttention(hidden_size, n_heads, kv_heads, head_dim, "a.", position_encoding=rope, qk_norm_eps=eps,
                        window=window)
    assert abs(part.scale - 1 / math.sqrt(head_dim)) < 1e-12
    w = Weights(part.tensor_specs(), dtype, std=0.15)
    part.load(w)
    pasts, news = [140, 3, 64], [30, 1, 66]
    x = [torch.randn(p + n, hidden_size).to(dtype) for p, n in zip(pasts, news)]
    want = plain_attention_part(np.concatenate([v.float().numpy() for v in x]), w.numpy, n_heads, kv_heads, head_dim,
                                eps, theta, part.scale, window, pasts, news)
    need = part.cache_need()
    assert need.kind == "kv" and need.window == window
    cache = SequenceCache({0: need}, 1024, dtype, DEVICE, K.page_size)
    cache.allocate()
    slots = [cache.alloc_slot() for _ in pasts]
    got = [[] for _ in pasts]
    for phase in (0, 1):
        entries, inputs = [], []
        for s, (p, n) in enumerate(zip(pasts, news)):
            lo, hi = (0, p) if phase == 0 else (p, p + n)
            entries.append(StepEntry(slots[s], [0] * (hi - lo), []))
            inputs.append(x[s][lo:hi])
        requests = [(entry.slot, len(entry.tokens)) for entry in entries]
        cache.reserve(requests)
        ctx, _, tables = build_step(K, dtype, DEVICE, cache, entries)
        residual = torch.zeros(ctx.n_rows, hidden_size, device=DEVICE)
        part.forward(ctx, torch.cat(inputs).to(DEVICE), residual, cache.layer_cache(0, True, tables))
        cache.commit(requests)
        at = 0
        for s, entry in enumerate(entries):
            got[s].append(residual[at:at + len(entry.tokens)].cpu().numpy())
            at += len(entry.tokens)
    for s in range(len(pasts)):
        assert schedules.relative_error(np.concatenate(got[s]), want[s]) < tol(dtype), s
    cache.check_invariants()
    if window:      # pages that left the window went back to the pool
        assert cache.groups[0].pages_of[slots[0]][0] == -1


@pytest.mark.parametrize("dtype", DTYPES)
def test_block_is_mixer_then_feed_forward_on_the_residual(K, dtype):
    hidden_size, n_heads, kv_heads, head_dim = 64, 4, 2, 16
    rope = RotaryEncoding(head_dim, 10000.0, 128)
    rope.build_tables(DEVICE)
    block = PreNormBlock(RMSNorm(hidden_size, 1e-6, "model.layers.0.input_layernorm.weight"),
                         GQAAttention(hidden_size, n_heads, kv_heads, head_dim, "model.layers.0.self_attn.",
                                      position_encoding=rope, qk_norm_eps=1e-6),
                         RMSNorm(hidden_size, 1e-6, "model.layers.0.post_attention_layernorm.weight"),
                         SwiGLU(hidden_size, 100, "model.layers.0.mlp."))
    w = Weights(block.tensor_specs(), dtype, std=0.15)
    block.load(w)
    cfg = plain.PlainConfig({"num_hidden_layers": 1, "hidden_size": hidden_size, "num_attention_heads": n_heads,
                             "num_key_value_heads": kv_heads, "head_dim": head_dim, "intermediate_size": 100,
                             "vocab_size": 10, "rms_norm_eps": 1e-6, "rope_theta": 10000.0})
    hidden = torch.randn(9, hidden_size)
    ctx, cache, tables, requests = make_ctx(K, dtype, {0: block.cache_need()}, [[0] * 9])
    residual = hidden.clone().to(DEVICE)
    block.forward(ctx, residual, cache.layer_cache(0, True, tables))
    assert rel(residual, plain.layer(cfg, w.numpy, 0, hidden.numpy())) < tol(dtype)


@pytest.fixture()
def toys():
    toy_parts.register()
    yield
    toy_parts.unregister()


# (the architecture with routing runs in float32 only: top-1 routing on rounded inputs may choose another expert
# than the plain form does)
@pytest.mark.parametrize("architecture,dtype", [(a, d) for a in ("ToyHybridForCausalLM", "ToyTwiceForCausalLM",
                                                                 "ToySharedCacheForCausalLM", "ToyParallelForCausalLM",
                                                                 "ToyWindowedForCausalLM")
                                                for d in ("float32", "bfloat16")]
                         + [("ToyOwnForCausalLM", "float32")])
def test_toy_architectures_on_the_gpu(toys, tmp_path, architecture, dtype):
    """A mixer with state of its own (whose decode steps are captured and replayed), a layer that runs twice, a
    layer that reads another layer's cache, a norm and an arrangement of a layer's parts of another make, layers
    whose attention sees a window of the keys beside layers that see all of them, and an
    architecture with a configuration class, tensor names, a routed feed-forward and a position encoding of its own: registered from the test, built, loaded and
    stepped by the unchanged engine."""
    folder = beholdd.write_random_model(str(tmp_path), toy_parts.config_dict(architecture), seed=3, dtype="bfloat16")
    toy_parts.check_architecture(architecture, folder, lambda f: Engine(f, dtype=dtype, max_tokens=1024),
                                 1e-4 if dtype == "float32" else 2e-2)
