"""Pins the plain implementation by what fixes it beside the reference's text: vectors that the
reference's own tests hold, special cases that reduce to a library routine, and invariants.
Each is chosen so that a plausible mistake fails it."""

import math

import numpy as np
import pytest
import scipy.special

import plain_qwen3 as plain

RNG = np.random.default_rng(1234)


# ---- RMSNorm -------------------------------------------------------------------------------

def test_rmsnorm_unit_rms_vector():
    # crates/beholdd-kernel/src/vecops.rs:204-210
    x = np.array([math.sin(i * 0.1) * 3.0 for i in range(512)], dtype=np.float32)
    y = plain.rmsnorm(x, None, 1e-6)
    assert abs(math.sqrt(float((y.astype(np.float64) ** 2).mean())) - 1.0) < 1e-4


def test_rmsnorm_applies_weight_vector():
    # crates/beholdd-kernel/src/vecops.rs:213-220: x already has unit rms, so y == w exactly
    y = plain.rmsnorm(np.ones(4, np.float32), np.array([2, 3, 4, 5], np.float32), 0.0)
    assert y.tolist() == [2.0, 3.0, 4.0, 5.0]


def test_rmsnorm_is_not_layernorm_and_weight_is_not_one_plus_w():
    x = RNG.normal(size=(3, 40)).astype(np.float32) + 2.0       # a mean that LayerNorm would remove
    w = RNG.normal(size=40).astype(np.float32)
    expected = x / np.sqrt((x.astype(np.float64) ** 2).mean(-1, keepdims=True) + 1e-5) * w
    assert np.allclose(plain.rmsnorm(x, w, 1e-5), expected, rtol=1e-6, atol=1e-7)
    assert not np.allclose(plain.rmsnorm(x, w, 1e-5), expected / w * (1 + w), atol=1e-3)


def test_rmsnorm_eps_is_inside_the_root():
    x = np.full(8, 1e-3, np.float32)
    y = plain.rmsnorm(x, None, 1e-2)
    assert np.allclose(y, 1e-3 / math.sqrt(1e-6 + 1e-2), rtol=1e-6)


# ---- softmax ---------------------------------------------------------------------------------

def test_softmax_vectors():
    # crates/beholdd-kernel/src/vecops.rs:223-248
    v = plain.softmax(np.array([1, 2, 3, -np.inf], np.float32))
    assert v[3] == 0.0 and abs(v.sum() - 1) < 1e-6 and v[2] > v[1] > v[0]
    assert (plain.softmax(np.full(4, -np.inf, np.float32)) == 0).all()
    big = plain.softmax(np.array([1000, 1001, 1002], np.float32))
    assert np.isfinite(big).all() and abs(big.sum() - 1) < 1e-6


def test_softmax_matches_scipy_and_is_shift_invariant():
    x = RNG.normal(size=(5, 33)).astype(np.float32) * 4
    assert np.allclose(plain.softmax(x), scipy.special.softmax(x.astype(np.float64), axis=-1), atol=1e-6)
    assert np.allclose(plain.softmax(x), plain.softmax(x + 7.5), atol=1e-6)


# ---- SiLU / SwiGLU ---------------------------------------------------------------------------

def test_silu_and_swiglu():
    assert plain.silu(np.float32(0)) == 0
    assert abs(float(plain.silu(np.float32(20))) - 20) < 1e-6
    g = RNG.normal(size=50).astype(np.float32) * 3
    u = RNG.normal(size=50).astype(np.float32)
    assert np.allclose(plain.swiglu(g, u), g * scipy.special.expit(g.astype(np.float64)) * u, atol=1e-6)
    # the gate is the FIRST argument: swapping the operands gives something else
    assert not np.allclose(plain.swiglu(g, u), plain.swiglu(u, g), atol=1e-3)


def test_swiglu_clamp_vector():
    # crates/beholdd-kernel/src/vecops.rs:251-260: gate clamped from above only, up both ways
    out = plain.swiglu(np.array([100, -100], np.float32), np.array([100, -100], np.float32), limit=10.0)
    assert abs(out[0] - float(plain.silu(np.float32(10))) * 10) < 1e-4
    assert abs(out[1] - float(plain.silu(np.float32(-100))) * -10) < 1e-4


# ---- RoPE --------------------------------------------------------------------------------------

def test_rope_split_half_vector():
    # crates/beholdd-kernel/src/vecops.rs:278-289
    x = np.array([1, 2, 3, 4], np.float32)
    assert plain.rope_split_half(x, [0, 0], [1, 1]).tolist() == [-3, -4, 1, 2]
    assert plain.rope_interleaved(x, [0, 0], [1, 1]).tolist() == [-2, 1, -4, 3]


def test_rope_round_trip_vector():
    # crates/beholdd-kernel/src/vecops.rs:292-304
    freqs = plain.rope_frequencies(1_000_000.0, 128)
    cos, sin = plain.rope_cos_sin(freqs, 1234)
    x = np.array([math.cos(i * 0.17) for i in range(128)], np.float32)
    y = plain.rope_split_half(x, cos, sin)
    assert not np.allclose(x, y)
    assert np.allclose(plain.rope_split_half(y, cos, sin, inverse=True), x, atol=1e-5)


def test_rope_is_a_complex_multiplication():
    hd, pos, theta = 32, 77, 10000.0
    x = RNG.normal(size=hd).astype(np.float32)
    freqs = plain.rope_frequencies(theta, hd)
    y = plain.rope_split_half(x, *plain.rope_cos_sin(freqs, pos))
    z = (x[:hd // 2] + 1j * x[hd // 2:]) * np.exp(1j * pos * freqs)
    assert np.allclose(y, np.concatenate([z.real, z.imag]), atol=1e-5)
    # frequencies fall with the index: 1, theta^(-2/hd), ...
    assert freqs[0] == 1.0 and np.isclose(freqs[1], theta ** (-2 / hd)) and np.isclose(freqs[-1], theta ** (-(hd - 2) / hd))


def test_rope_position_zero_is_identity_and_scores_depend_on_distance_only():
    hd = 16
    freqs = plain.rope_frequencies(10000.0, hd)
    q, k = RNG.normal(size=hd).astype(np.float32), RNG.normal(size=hd).astype(np.float32)
    assert np.array_equal(plain.rope_split_half(q, *plain.rope_cos_sin(freqs, 0)), q)

    def score(a, b):
        return float(plain.rope_split_half(q, *plain.rope_cos_sin(freqs, a)) @ plain.rope_split_half(k, *plain.rope_cos_sin(freqs, b)))

    assert abs(score(9, 4) - score(109, 104)) < 1e-4
    assert abs(score(9, 4) - score(4, 9)) > 1e-3          # the sign of the distance matters


# ---- attention -----------------------------------------------------------------------------------

def test_attention_known_softmax_vector():
    # crates/beholdd-backend/src/cpu.rs:1389-1411
    out = plain.causal_attention(np.array([[1, 0], [1, 0]], np.float32), np.array([[0, 0], [math.log(3), 0]], np.float32),
                                 np.array([[2, 4], [6, 8]], np.float32), 1, 1, 2, 1.0)
    assert np.allclose(out, [[2, 4], [5, 7]], atol=1e-6)


def test_attention_mask_and_gqa_vector():
    # crates/beholdd-backend/src/cpu.rs:1414-1440: contiguous groups, the future excluded
    out = plain.causal_attention(np.zeros((2, 4), np.float32), np.zeros((2, 2), np.float32),
                                 np.array([[1, 10], [3, 30]], np.float32), 4, 2, 1, 1.0)
    assert out.tolist() == [[1, 1, 10, 10], [2, 2, 20, 20]]


def test_attention_incremental_vector():
    # crates/beholdd-backend/src/cpu.rs:1544-1570: the query stands at position 1 of 3 cached keys
    out = plain.causal_attention(np.array([[1]], np.float32), np.array([[0], [math.log(3)], [100]], np.float32),
                                 np.array([[2], [6], [10000]], np.float32), 1, 1, 1, 1.0, query_start=1)
    assert abs(out[0, 0] - 5.0) < 1e-6


def test_attention_reduces_to_plain_softmax_attention():
    t, h, hd = 7, 3, 8
    q, k, v = (RNG.normal(size=(t, h * hd)).astype(np.float32) for _ in range(3))
    scale = 1 / math.sqrt(hd)
    out = plain.causal_attention(q, k, v, h, h, hd, scale).reshape(t, h, hd)
    for head in range(h):
        qq, kk, vv = (a.reshape(t, h, hd)[:, head].astype(np.float64) for a in (q, k, v))
        scores = qq @ kk.T * scale
        scores[np.triu_indices(t, 1)] = -np.inf
        assert np.allclose(out[:, head], scipy.special.softmax(scores, -1) @ vv, atol=1e-5)


def test_attention_single_position_repeats_values_per_group():
    # the trick tools/qwen3_dense_ref.py:65-69 relies on
    v = RNG.normal(size=(1, 2 * 4)).astype(np.float32)
    out = plain.causal_attention(RNG.normal(size=(1, 6 * 4)).astype(np.float32), RNG.normal(size=(1, 8)).astype(np.float32),
                                 v, 6, 2, 4, 0.5).reshape(6, 4)
    assert np.allclose(out[:3], v.reshape(2, 4)[0]) and np.allclose(out[3:], v.reshape(2, 4)[1])


def test_attention_future_never_changes_the_past():
    t, hd = 6, 4
    q, k, v = (RNG.normal(size=(t, 2 * hd)).astype(np.float32) for _ in range(3))
    whole = plain.causal_attention(q, k, v, 2, 2, hd, 0.5)
    assert np.array_equal(whole[:4], plain.causal_attention(q[:4], k[:4], v[:4], 2, 2, hd, 0.5))


# ---- linear, embedding, greedy ------------------------------------------------------------------

def test_linear_vector_and_orientation():
    # crates/beholdd-kernel/src/bf16.rs:181-190
    assert plain.linear(np.array([3, 5, 8, 0.25], np.float32), np.array([[1, 2, -0.5, 4]], np.float32))[0] == 10.0
    w = RNG.normal(size=(5, 3)).astype(np.float32)      # [out, in]
    x = RNG.normal(size=(2, 3)).astype(np.float32)
    assert plain.linear(x, w).shape == (2, 5)
    assert np.allclose(plain.linear(x, w), x @ w.T, atol=1e-6)


def test_greedy_vectors():
    # crates/beholdd-model/src/qwen3moe/forward.rs:2257-2262
    assert plain.greedy_token([-1, 3, 3, 2]) == 1
    for bad in ([], [0, float("nan")], [float("inf"), 0]):
        with pytest.raises(ValueError):
            plain.greedy_token(bad)


# ---- the whole model ---------------------------------------------------------------------------------

def _tiny_weights(cfg, rng, identity=False):
    w = {}
    d, hd, nh, nkv, f, v = cfg.hidden, cfg.head_dim, cfg.n_heads, cfg.n_kv_heads, cfg.intermediate, cfg.vocab
    w["model.embed_tokens.weight"] = rng.normal(size=(v, d)).astype(np.float32) * 0.5
    for i in range(cfg.n_layers):
        p = f"model.layers.{i}."
        w[p + "input_layernorm.weight"] = 1 + rng.normal(size=d).astype(np.float32) * 0.1
        w[p + "post_attention_layernorm.weight"] = 1 + rng.normal(size=d).astype(np.float32) * 0.1
        w[p + "self_attn.q_proj.weight"] = rng.normal(size=(nh * hd, d)).astype(np.float32) * 0.2
        w[p + "self_attn.k_proj.weight"] = rng.normal(size=(nkv * hd, d)).astype(np.float32) * 0.2
        w[p + "self_attn.v_proj.weight"] = rng.normal(size=(nkv * hd, d)).astype(np.float32) * 0.2
        w[p + "self_attn.o_proj.weight"] = rng.normal(size=(d, nh * hd)).astype(np.float32) * 0.2
        w[p + "self_attn.q_norm.weight"] = 1 + rng.normal(size=hd).astype(np.float32) * 0.1
        w[p + "self_attn.k_norm.weight"] = 1 + rng.normal(size=hd).astype(np.float32) * 0.1
        w[p + "mlp.gate_proj.weight"] = rng.normal(size=(f, d)).astype(np.float32) * 0.2
        w[p + "mlp.up_proj.weight"] = rng.normal(size=(f, d)).astype(np.float32) * 0.2
        w[p + "mlp.down_proj.weight"] = rng.normal(size=(d, f)).astype(np.float32) * 0.2
    w["model.norm.weight"] = 1 + rng.normal(size=d).astype(np.float32) * 0.1
    w["lm_head.weight"] = rng.normal(size=(v, d)).astype(np.float32) * 0.2
    return w


def _cfg(**over):
    base = {"num_hidden_layers": 2, "hidden_size": 12, "num_attention_heads": 4, "num_key_value_heads": 2,
            "head_dim": 4, "intermediate_size": 10, "vocab_size": 17, "rms_norm_eps": 1e-6, "rope_theta": 100.0,
            "tie_word_embeddings": False}
    base.update(over)
    return plain.PlainConfig(base)


def test_model_is_causal_and_deterministic():
    cfg = _cfg()
    w = _tiny_weights(cfg, np.random.default_rng(5))
    tokens = [3, 1, 4, 1, 5, 9, 2, 6]
    whole = plain.forward_logits(cfg, w, tokens)
    assert np.array_equal(whole, plain.forward_logits(cfg, w, tokens))
    assert np.allclose(whole[:5], plain.forward_logits(cfg, w, tokens[:5]), atol=1e-6)


def test_tied_head_equals_untied_head_with_the_embedding():
    cfg_untied, cfg_tied = _cfg(), _cfg(tie_word_embeddings=True)
    w = _tiny_weights(cfg_untied, np.random.default_rng(6))
    w["lm_head.weight"] = w["model.embed_tokens.weight"].copy()
    assert np.array_equal(plain.forward_logits(cfg_untied, w, [1, 2, 3]), plain.forward_logits(cfg_tied, w, [1, 2, 3]))


def test_hand_checkable_model_logits_equal_hidden_over_rms():
    # In the manner of crates/beholdd-model/src/qwen3moe/forward.rs:2808-2851: with zero output
    # projections the layers add nothing, so logits = lm_head * (embedding / rms).
    cfg = _cfg(num_hidden_layers=1)
    w = _tiny_weights(cfg, np.random.default_rng(7))
    w["model.layers.0.self_attn.o_proj.weight"][:] = 0
    w["model.layers.0.mlp.down_proj.weight"][:] = 0
    w["model.norm.weight"][:] = 1
    logits = plain.forward_logits(cfg, w, [2, 5])
    e = w["model.embed_tokens.weight"][[2, 5]].astype(np.float64)
    expected = (e / np.sqrt((e ** 2).mean(-1, keepdims=True) + 1e-6)) @ w["lm_head.weight"].astype(np.float64).T
    assert np.allclose(logits, expected, atol=1e-5)


def test_greedy_generate_stop_token_is_not_emitted():
    cfg = _cfg()
    w = _tiny_weights(cfg, np.random.default_rng(9))
    tokens, stop = plain.greedy_generate(cfg, w, [1, 2, 3], 6)
    assert len(tokens) == 6 and stop is None
    again, stop = plain.greedy_generate(cfg, w, [1, 2, 3], 6, stop_tokens=(tokens[2],))
    first = tokens.index(tokens[2])
    assert again == tokens[:first] and stop == tokens[2]
