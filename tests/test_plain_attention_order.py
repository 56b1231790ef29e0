"""What fixes the order of operations inside the plain implementation's attention block and layer,
beside the reading of the reference's text: a regression vector that the reference's own test holds,
a special case with a closed form, and the shift invariance of rotary attention.  Every check comes
with mutated copies of the block (one plausible mistake each) that must fail it, so that the check is
known to have teeth; the unmutated copy is bit-equal to the plain implementation's block."""

import math

import numpy as np
import pytest
import scipy.special

import plain_qwen3 as plain

F32 = np.float32


def _block(cfg, w, prefix, hidden, first_position=0, mistake=None):
    """The arrangement of plain.attention_block from the same part functions, with one mistake switched on."""
    t_len, hd, nh, nkv = hidden.shape[0], cfg.head_dim, cfg.n_heads, cfg.n_kv_heads
    xn = plain.rmsnorm(hidden, w[prefix + "input_layernorm.weight"], cfg.eps)
    if mistake == "no input norm":
        xn = hidden
    q = plain.linear(xn, w[prefix + "self_attn.q_proj.weight"]).reshape(t_len, nh, hd)
    k = plain.linear(xn, w[prefix + "self_attn.k_proj.weight"]).reshape(t_len, nkv, hd)
    v = plain.linear(xn, w[prefix + "self_attn.v_proj.weight"])
    wq, wk = w[prefix + "self_attn.q_norm.weight"], w[prefix + "self_attn.k_norm.weight"]
    if mistake == "q and k norm weights swapped":
        wq, wk = wk, wq
    eps = 1e-6 if mistake == "an epsilon of their own for the head norms" else cfg.eps
    freqs = plain.rope_frequencies(cfg.theta, hd)
    rotate = plain.rope_interleaved if mistake == "adjacent pairs" else plain.rope_split_half

    def rotated(x):
        out = x.copy()
        for t in range(t_len):
            cos, sin = plain.rope_cos_sin(freqs, first_position + t)
            out[t] = rotate(x[t], cos, sin, inverse=(mistake == "rotation the other way"))
        return out

    if mistake == "norm after the rotation":
        q, k = plain.rmsnorm(rotated(q), wq, eps), plain.rmsnorm(rotated(k), wk, eps)
    elif mistake == "no head norms":
        q, k = rotated(q), rotated(k)
    elif mistake == "values normed too":
        q, k = rotated(plain.rmsnorm(q, wq, eps)), rotated(plain.rmsnorm(k, wk, eps))
        v = plain.rmsnorm(v.reshape(t_len, nkv, hd), wk, eps).reshape(t_len, nkv * hd)
    else:
        q, k = rotated(plain.rmsnorm(q, wq, eps)), rotated(plain.rmsnorm(k, wk, eps))
    scale = F32(1.0) / np.sqrt(F32(hd))
    if mistake == "scale 1/head_dim":
        scale = F32(1.0) / F32(hd)
    attended = plain.causal_attention(q.reshape(t_len, nh * hd), k.reshape(t_len, nkv * hd), v, nh, nkv, hd, scale)
    out = plain.linear(attended, w[prefix + "self_attn.o_proj.weight"])
    return out.astype(F32) if mistake == "no residual" else (hidden + out).astype(F32)


def _random_block(cfg, rng, spread=0.5):
    """Weights of one attention block whose norm vectors are far from one and from each other."""
    d, hd, nh, nkv = cfg.hidden, cfg.head_dim, cfg.n_heads, cfg.n_kv_heads
    p = "model.layers.0."
    return p, {
        p + "input_layernorm.weight": (1 + spread * rng.normal(size=d)).astype(F32),
        p + "self_attn.q_proj.weight": rng.normal(size=(nh * hd, d)).astype(F32),
        p + "self_attn.k_proj.weight": rng.normal(size=(nkv * hd, d)).astype(F32),
        p + "self_attn.v_proj.weight": rng.normal(size=(nkv * hd, d)).astype(F32),
        p + "self_attn.o_proj.weight": rng.normal(size=(d, nh * hd)).astype(F32),
        p + "self_attn.q_norm.weight": (1 + spread * rng.normal(size=hd)).astype(F32),
        p + "self_attn.k_norm.weight": (1 + spread * rng.normal(size=hd)).astype(F32),
    }


def _cfg(**over):
    base = {"num_hidden_layers": 1, "hidden_size": 12, "num_attention_heads": 4, "num_key_value_heads": 2,
            "head_dim": 6, "intermediate_size": 10, "vocab_size": 17, "rms_norm_eps": 1e-6, "rope_theta": 100.0}
    base.update(over)
    return plain.PlainConfig(base)


def test_the_unmutated_copy_is_the_plain_block():
    cfg = _cfg()
    prefix, w = _random_block(cfg, np.random.default_rng(0))
    hidden = np.random.default_rng(1).normal(size=(7, cfg.hidden)).astype(F32)
    for first in (0, 5):
        assert np.array_equal(_block(cfg, w, prefix, hidden, first), plain.attention_block(cfg, w, prefix, hidden, first))


# ---- 1. the regression vector of the reference's tiny hand-authored block -----------------------------

# crates/beholdd-model/src/qwen3moe/forward.rs:3557-3734 writes the fixture: width 4, one head of 4, identity q
# and k projections, v = 0.5 I, o = I, every norm weight one, eps 1e-6, theta 10000, embedding rows
# [1, -0.5, 0.25, 2] and [-0.75, 1.5, 0.5, -1]; its routed feed-forward sends token 0 to expert 0
# (gate I, up I, down 0.25 I) and token 1 to expert 1 (gate -I, up 0.75 I, down -0.5 I), each with weight one
# (:2310-2311).  :2338-2353 holds the block's output for tokens [0, 1] to 1e-6.
FIXTURE_EMBEDDING = np.array([[1.0, -0.5, 0.25, 2.0], [-0.75, 1.5, 0.5, -1.0]], F32)
FIXTURE_BLOCK_OUTPUT = np.array([1.566_429_5, -0.698_426_66, 0.364_983_08, 3.507_802_2,
                                 -0.960_466_3, 2.371_297, 0.779_807_2, -1.195_086_2], F32)


def _fixture():
    cfg = _cfg(hidden_size=4, num_attention_heads=1, num_key_value_heads=1, head_dim=4, intermediate_size=4,
               vocab_size=2, rope_theta=10000.0)
    eye, ones, p = np.eye(4, dtype=F32), np.ones(4, F32), "model.layers.0."
    w = {p + "input_layernorm.weight": ones, p + "post_attention_layernorm.weight": ones,
         p + "self_attn.q_proj.weight": eye, p + "self_attn.k_proj.weight": eye,
         p + "self_attn.v_proj.weight": 0.5 * eye, p + "self_attn.o_proj.weight": eye,
         p + "self_attn.q_norm.weight": ones, p + "self_attn.k_norm.weight": ones}
    return cfg, w, p


def _fixture_feed_forward(cfg, w, prefix, hidden, parallel_to=None):
    """The fixture's two one-expert feed-forwards on the normed residual, added to it."""
    x = plain.rmsnorm(hidden if parallel_to is None else parallel_to, w[prefix + "post_attention_layernorm.weight"], cfg.eps)
    out = hidden.copy()
    out[0] += F32(0.25) * plain.swiglu(x[0], x[0])
    out[1] += F32(-0.5) * plain.swiglu(-x[1], F32(0.75) * x[1])
    return out


def test_regression_vector_of_the_reference_fixture():
    cfg, w, p = _fixture()
    hidden = plain.attention_block(cfg, w, p, FIXTURE_EMBEDDING)
    out = _fixture_feed_forward(cfg, w, p, hidden)
    assert np.abs(out.ravel() - FIXTURE_BLOCK_OUTPUT).max() < 1e-6


@pytest.mark.parametrize("mistake", ["scale 1/head_dim", "adjacent pairs", "rotation the other way",
                                     "no input norm", "no residual", "values normed too"])
def test_regression_vector_rejects_a_wrong_attention_block(mistake):
    # (the fixture's head norms see vectors of unit rms and unit weights, so it cannot tell whether they
    # are there or where; the closed form below does that)
    cfg, w, p = _fixture()
    out = _fixture_feed_forward(cfg, w, p, _block(cfg, w, p, FIXTURE_EMBEDDING, mistake=mistake))
    assert np.abs(out.ravel() - FIXTURE_BLOCK_OUTPUT).max() > 1e-4, mistake      # a hundred times the vector's tolerance


def test_regression_vector_rejects_a_wrong_layer_order():
    cfg, w, p = _fixture()
    # feed-forward first, then attention
    swapped = plain.attention_block(cfg, w, p, _fixture_feed_forward(cfg, w, p, FIXTURE_EMBEDDING))
    assert np.abs(swapped.ravel() - FIXTURE_BLOCK_OUTPUT).max() > 1e-4
    # both halves read the layer's input (a parallel block)
    attended = plain.attention_block(cfg, w, p, FIXTURE_EMBEDDING)
    parallel = _fixture_feed_forward(cfg, w, p, attended, parallel_to=FIXTURE_EMBEDDING)
    assert np.abs(parallel.ravel() - FIXTURE_BLOCK_OUTPUT).max() > 1e-4


# ---- 2. one head of two dimensions: a closed form ---------------------------------------------------------

def _closed_form_case():
    """One head of size two (a single rotary pair of frequency one), q norm weight [a, 0], k norm weight [b, c],
    a large epsilon.  With q^ = q / sqrt(mean(q^2) + eps) and k^ likewise, the rotated query at position m is
    a q^_0 (cos m, sin m), so its score against the key at position n is
        a q^_0 (b k^_0 cos(m - n) + c k^_1 sin(m - n)) / sqrt(2),
    which a wrong order, swapped weights or another epsilon all change."""
    cfg = _cfg(hidden_size=2, num_attention_heads=1, num_key_value_heads=1, head_dim=2, rms_norm_eps=0.25, rope_theta=77.0)
    rng = np.random.default_rng(11)
    eye, p = np.eye(2, dtype=F32), "model.layers.0."
    w = {p + "input_layernorm.weight": np.ones(2, F32),
         p + "self_attn.q_proj.weight": rng.normal(size=(2, 2)).astype(F32), p + "self_attn.k_proj.weight": rng.normal(size=(2, 2)).astype(F32),
         p + "self_attn.v_proj.weight": rng.normal(size=(2, 2)).astype(F32), p + "self_attn.o_proj.weight": eye,
         p + "self_attn.q_norm.weight": np.array([1.7, 0.0], F32), p + "self_attn.k_norm.weight": np.array([0.6, -1.3], F32)}
    hidden = rng.normal(size=(5, 2)).astype(F32)
    return cfg, w, p, hidden


def _closed_form_expected(cfg, w, p, hidden, first_position):
    eps = cfg.eps
    x = hidden.astype(np.float64)
    xn = x / np.sqrt((x * x).mean(-1, keepdims=True) + eps)
    q, k, v = (xn @ w[p + f"self_attn.{name}_proj.weight"].astype(np.float64).T for name in "qkv")
    qh = q / np.sqrt((q * q).mean(-1, keepdims=True) + eps)
    kh = k / np.sqrt((k * k).mean(-1, keepdims=True) + eps)
    a = float(w[p + "self_attn.q_norm.weight"][0])
    b, c = (float(t) for t in w[p + "self_attn.k_norm.weight"])
    out = x.copy()
    for m in range(len(x)):
        delta = np.arange(m + 1)[::-1].astype(np.float64)        # m - n for n = 0..m; the first position cancels
        scores = a * qh[m, 0] * (b * kh[:m + 1, 0] * np.cos(delta) + c * kh[:m + 1, 1] * np.sin(delta)) / math.sqrt(2.0)
        out[m] += scipy.special.softmax(scores) @ v[:m + 1]
    return out


@pytest.mark.parametrize("first_position", [0, 9])
def test_closed_form_of_a_single_rotary_pair(first_position):
    cfg, w, p, hidden = _closed_form_case()
    got = plain.attention_block(cfg, w, p, hidden, first_position)
    assert np.abs(got - _closed_form_expected(cfg, w, p, hidden, first_position)).max() < 2e-6


@pytest.mark.parametrize("mistake", ["norm after the rotation", "q and k norm weights swapped",
                                     "an epsilon of their own for the head norms", "rotation the other way",
                                     "scale 1/head_dim", "no head norms"])
def test_closed_form_rejects_a_wrong_attention_block(mistake):
    cfg, w, p, hidden = _closed_form_case()
    got = _block(cfg, w, p, hidden, 0, mistake=mistake)
    assert np.abs(got - _closed_form_expected(cfg, w, p, hidden, 0)).max() > 1e-3, mistake


# ---- 3. only distances count ---------------------------------------------------------------------------------

def test_a_shift_of_all_positions_changes_nothing():
    cfg = _cfg()
    prefix, w = _random_block(cfg, np.random.default_rng(3))
    hidden = np.random.default_rng(4).normal(size=(9, cfg.hidden)).astype(F32)
    base = plain.attention_block(cfg, w, prefix, hidden, 0)
    for shift in (1, 37, 1000):
        assert np.abs(plain.attention_block(cfg, w, prefix, hidden, shift) - base).max() < 2e-5 * np.abs(base).max()
    # a head norm applied after the rotation, with weights that differ within a pair, breaks it
    wrong = [_block(cfg, w, prefix, hidden, shift, mistake="norm after the rotation") for shift in (0, 37)]
    assert np.abs(wrong[1] - wrong[0]).max() > 1e-2 * np.abs(base).max()


def test_the_whole_model_is_shift_invariant_too():
    cfg = plain.PlainConfig({"num_hidden_layers": 2, "hidden_size": 12, "num_attention_heads": 4, "num_key_value_heads": 2,
                             "head_dim": 6, "intermediate_size": 10, "vocab_size": 17, "rms_norm_eps": 1e-5,
                             "rope_theta": 100.0, "tie_word_embeddings": True})
    rng = np.random.default_rng(5)
    w = {"model.embed_tokens.weight": rng.normal(size=(17, 12)).astype(F32), "model.norm.weight": (1 + 0.3 * rng.normal(size=12)).astype(F32)}
    for index in range(2):
        _, block = _random_block(cfg, rng, spread=0.3)
        p = f"model.layers.{index}."
        w.update({name.replace("model.layers.0.", p): value for name, value in block.items()})
        w[p + "post_attention_layernorm.weight"] = (1 + 0.3 * rng.normal(size=12)).astype(F32)
        w[p + "mlp.gate_proj.weight"] = rng.normal(size=(10, 12)).astype(F32) * 0.3
        w[p + "mlp.up_proj.weight"] = rng.normal(size=(10, 12)).astype(F32) * 0.3
        w[p + "mlp.down_proj.weight"] = rng.normal(size=(12, 10)).astype(F32) * 0.3
    tokens = [3, 1, 4, 1, 5, 9, 2, 6]
    base = plain.forward_logits(cfg, w, tokens)
    moved = plain.forward_logits(cfg, w, tokens, first_position=123)
    assert np.abs(moved - base).max() < 5e-5 * np.abs(base).max()
