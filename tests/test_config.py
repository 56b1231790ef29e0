"""The typed configuration and the registry."""

import json

import pytest

import beholdd
from beholdd.config import ConfigError, Qwen3Config, read_config_json


def test_every_number_comes_from_the_file(tiny_configs):
    for name in ("A", "B"):
        raw = tiny_configs[name]
        cfg = Qwen3Config.from_dict(raw)
        assert (cfg.n_layers, cfg.hidden, cfg.n_heads, cfg.n_kv_heads, cfg.head_dim) == (
            raw["num_hidden_layers"], raw["hidden_size"], raw["num_attention_heads"], raw["num_key_value_heads"],
            raw["head_dim"])
        assert (cfg.intermediate, cfg.vocab, cfg.rms_eps, cfg.rope_theta, cfg.max_position, cfg.tie_word_embeddings) == (
            raw["intermediate_size"], raw["vocab_size"], raw["rms_norm_eps"], raw["rope_theta"],
            raw["max_position_embeddings"], raw["tie_word_embeddings"])
        assert cfg.q_width == cfg.n_heads * cfg.head_dim and cfg.kv_width == cfg.n_kv_heads * cfg.head_dim
        assert Qwen3Config.from_dict(cfg.to_dict()) == cfg
    b = Qwen3Config.from_dict(tiny_configs["B"])
    assert b.q_width == 256 != b.hidden and b.group == 4


@pytest.mark.parametrize("key", ["num_hidden_layers", "hidden_size", "num_attention_heads", "num_key_value_heads",
                                 "intermediate_size", "vocab_size", "rms_norm_eps", "rope_theta",
                                 "max_position_embeddings"])
def test_a_missing_key_is_an_error_not_a_default(tiny_configs, key):
    raw = tiny_configs["A"]
    del raw[key]
    with pytest.raises(ConfigError, match=key):
        Qwen3Config.from_dict(raw)


def test_head_dim_defaults_only_when_it_divides(tiny_configs):
    raw = tiny_configs["A"]
    del raw["head_dim"]
    assert Qwen3Config.from_dict(raw).head_dim == 16
    raw["num_attention_heads"], raw["num_key_value_heads"] = 3, 3
    with pytest.raises(ConfigError, match="head_dim"):
        Qwen3Config.from_dict(raw)


@pytest.mark.parametrize("change,message", [
    ({"num_attention_heads": 6, "num_key_value_heads": 4}, "6 query heads do not group evenly into 4 kv heads"),
    ({"head_dim": 15}, "even"),
    ({"rms_norm_eps": 0.0}, "epsilon"),
    ({"rms_norm_eps": -1e-6}, "epsilon"),
    ({"rope_theta": 0}, "RoPE base"),
    ({"num_hidden_layers": 0}, "at least 1"),
    ({"num_hidden_layers": 2 ** 40}, "at most"),         # (a list of that many layers would never be finished)
    ({"hidden_size": 2 ** 31}, "at most"),               # the kernels take 32-bit sizes
    ({"vocab_size": "many"}, "integer"),
    ({"hidden_size": 64.5}, "integer"),
    ({"attention_bias": True}, "attention_bias"),
    ({"hidden_act": "gelu"}, "hidden_act"),
    ({"use_sliding_window": True, "sliding_window": 128}, "sliding"),
    ({"rope_scaling": {"rope_type": "yarn", "factor": 4.0}}, "scaling"),
    ({"layer_types": ["full_attention", "sliding_attention"]}, "sliding_attention"),
    ({"model_type": "llama"}, "model_type"),
    ({"tie_word_embeddings": "yes"}, "true or false"),
    ({"eos_token_id": 100000}, "outside the vocabulary"),
])
def test_refusals(tiny_configs, change, message):
    raw = dict(tiny_configs["A"], **change)
    with pytest.raises(ConfigError, match=message):
        Qwen3Config.from_dict(raw)


def test_harmless_keys_are_ignored_and_equivalent_spellings_accepted(tiny_configs):
    raw = dict(tiny_configs["B"], torch_dtype="bfloat16", bos_token_id=1, eos_token_id=[2, 3], use_cache=True,
               sliding_window=None, use_sliding_window=False, max_window_layers=3, rope_scaling=None,
               layer_types=["full_attention"] * 3, attention_dropout=0.0, transformers_version="4.51.0")
    cfg = Qwen3Config.from_dict(raw)
    assert cfg.eos_token_ids == (2, 3)
    moved = dict(tiny_configs["B"])
    del moved["rope_theta"]
    moved["rope_parameters"] = {"rope_type": "default", "rope_theta": 1000000.0}
    assert Qwen3Config.from_dict(moved).rope_theta == 1000000.0


def test_registry_resolves_by_exact_name(tmp_path, tiny_configs):
    entry = beholdd.resolve_architecture(tiny_configs["A"])
    assert entry.name == "Qwen3ForCausalLM" and entry.config_class is Qwen3Config
    for names in (["Qwen3MoeForCausalLM"], ["qwen3forcausallm"], [], ["Qwen3ForCausalLM", "Other"], None):
        with pytest.raises(ConfigError):
            beholdd.resolve_architecture(dict(tiny_configs["A"], architectures=names))
    (tmp_path / "config.json").write_text("{not json")
    with pytest.raises(ConfigError, match="JSON"):
        read_config_json(str(tmp_path))
    with pytest.raises(ConfigError, match="no such file"):
        read_config_json(str(tmp_path / "missing"))
    (tmp_path / "config.json").write_text(json.dumps([1, 2]))
    with pytest.raises(ConfigError, match="object"):
        read_config_json(str(tmp_path))


def test_the_model_is_built_from_the_configuration_layer_by_layer(tiny_configs):
    cfg = Qwen3Config.from_dict(tiny_configs["B"])
    model = beholdd.resolve_architecture(tiny_configs["B"]).build(cfg)
    assert len(model.blocks) == 3 and model.schedule == [(0, 0), (1, 1), (2, 2)]
    mixer = model.blocks[1].mixer
    assert (mixer.n_heads, mixer.n_kv_heads, mixer.head_dim, mixer.qk_norm_eps) == (8, 2, 32, 1e-5)
    assert model.blocks[2].feed_forward.intermediate == 160 and model.final_norm.eps == 1e-5
    names = [s.name for s in model.tensor_specs()]
    assert len(names) == 11 * 3 + 3 and "lm_head.weight" in names          # 11 per layer + embedding, norm, head
    tied = beholdd.resolve_architecture(tiny_configs["A"]).build(Qwen3Config.from_dict(tiny_configs["A"]))
    assert len(tied.tensor_specs()) == 11 * 2 + 2 and tied.head.tied_to is tied.embedding
