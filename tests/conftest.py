import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
for path in (ROOT, os.path.dirname(os.path.abspath(__file__))):
    if path not in sys.path:
        sys.path.insert(0, path)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs an MI355X (run with -m gpu)")


# Two tiny Qwen3 configurations that differ in every size and option.
TINY_A = {
    "architectures": ["Qwen3ForCausalLM"], "model_type": "qwen3",
    "num_hidden_layers": 2, "hidden_size": 64, "num_attention_heads": 4, "num_key_value_heads": 2,
    "head_dim": 16, "intermediate_size": 128, "vocab_size": 256, "rope_theta": 10000.0,
    "rms_norm_eps": 1e-6, "max_position_embeddings": 128, "tie_word_embeddings": True,
    "hidden_act": "silu", "attention_bias": False,
}
TINY_B = {
    "architectures": ["Qwen3ForCausalLM"], "model_type": "qwen3",
    "num_hidden_layers": 3, "hidden_size": 96, "num_attention_heads": 8, "num_key_value_heads": 2,
    "head_dim": 32, "intermediate_size": 160, "vocab_size": 384, "rope_theta": 1000000.0,
    "rms_norm_eps": 1e-5, "max_position_embeddings": 256, "tie_word_embeddings": False,
    "hidden_act": "silu", "attention_bias": False,
}
# A third one for the GPU tests: sizes that are no power of two, a head size of 48, one kv head
# per three query heads, a long context.
TINY_C = {
    "architectures": ["Qwen3ForCausalLM"], "model_type": "qwen3",
    "num_hidden_layers": 2, "hidden_size": 120, "num_attention_heads": 6, "num_key_value_heads": 2,
    "head_dim": 48, "intermediate_size": 200, "vocab_size": 331, "rope_theta": 50000.0,
    "rms_norm_eps": 1e-5, "max_position_embeddings": 1024, "tie_word_embeddings": False,
    "hidden_act": "silu", "attention_bias": False,
}
# The head size and group of the large models (128, four query heads per kv head), small otherwise.
TINY_D = {
    "architectures": ["Qwen3ForCausalLM"], "model_type": "qwen3",
    "num_hidden_layers": 2, "hidden_size": 320, "num_attention_heads": 8, "num_key_value_heads": 2,
    "head_dim": 128, "intermediate_size": 896, "vocab_size": 1500, "rope_theta": 1000000.0,
    "rms_norm_eps": 1e-6, "max_position_embeddings": 2048, "tie_word_embeddings": True,
    "hidden_act": "silu", "attention_bias": False,
}
# Seventeen query heads to a kv head: beyond what the decode attention that starts from the projection rows takes,
# so decode steps run the norm-rotate-write kernel and the attention kernel one after the other.
TINY_E = {
    "architectures": ["Qwen3ForCausalLM"], "model_type": "qwen3",
    "num_hidden_layers": 1, "hidden_size": 72, "num_attention_heads": 34, "num_key_value_heads": 2,
    "head_dim": 64, "intermediate_size": 100, "vocab_size": 211, "rope_theta": 10000.0,
    "rms_norm_eps": 1e-6, "max_position_embeddings": 512, "tie_word_embeddings": False,
    "hidden_act": "silu", "attention_bias": False,
}
CONFIGS = {"A": TINY_A, "B": TINY_B, "C": TINY_C, "D": TINY_D, "E": TINY_E}


@pytest.fixture()
def tiny_configs():
    import copy
    return copy.deepcopy(CONFIGS)


@pytest.fixture(scope="session")
def model_dirs(tmp_path_factory):
    """Model folders with seeded random weights, made once per session in a temporary place.
    Key: (config name, storage dtype)."""
    import beholdd

    made = {}

    def get(name: str, dtype: str = "bfloat16", seed: int = 0, std: float = 0.02):
        key = (name, dtype, seed, std)
        if key not in made:
            folder = tmp_path_factory.mktemp(f"tiny_{name}_{dtype}_{seed}")
            config = CONFIGS[name]
            beholdd.write_random_model(str(folder), dict(config), seed=seed, dtype=dtype, std=std)
            made[key] = str(folder)
        return made[key]

    return get
