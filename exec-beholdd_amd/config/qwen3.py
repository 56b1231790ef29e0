"""Qwen3 dense: the typed configuration read from config.json.

Fields and checks follow the reference's `Config` (crates/beholdd-model/src/qwen3moe.rs:124-154,
validation :235-289): every semantic number is required, head counts must group evenly, the
head size must be even, and switches this architecture does not implement (biases, a sliding
window in use, scaled rotation) are refused rather than ignored (:1145-1178).
"""

from __future__ import annotations

from dataclasses import dataclass, field

from .base import ConfigError, ConfigReader, LayerKinds


@dataclass(frozen=True)
class Qwen3Config:
    architecture: str
    n_layers: int
    hidden: int
    n_heads: int
    n_kv_heads: int
    head_dim: int
    intermediate: int
    vocab: int
    rms_eps: float
    rope_theta: float
    max_position: int
    tie_word_embeddings: bool
    eos_token_ids: tuple = field(default_factory=tuple)

    # ---- derived ----
    @property
    def q_width(self) -> int:
        return self.n_heads * self.head_dim

    @property
    def kv_width(self) -> int:
        return self.n_kv_heads * self.head_dim

    @property
    def group(self) -> int:
        return self.n_heads // self.n_kv_heads

    def layer_kinds(self) -> list[LayerKinds]:
        """Layer by layer, the names of the parts.  Qwen3 dense is uniform."""
        kinds = LayerKinds(mixer="gqa_attention", feed_forward="swiglu", norm="rmsnorm", block="pre_norm")
        return [kinds for _ in range(self.n_layers)]

    def schedule(self) -> list[tuple[int, int]]:
        """The order in which layers run: (layer index, cache entry index) pairs."""
        return [(index, index) for index in range(self.n_layers)]

    # ---- reading ----
    @classmethod
    def from_dict(cls, data: dict, origin: str = "config.json") -> "Qwen3Config":
        r = ConfigReader(data, origin)
        names = data.get("architectures")
        architecture = names[0] if isinstance(names, list) and names else "Qwen3ForCausalLM"

        n_layers = r.integer("num_hidden_layers", minimum=1, maximum=1 << 20)      # (a part object and a cache entry each)
        hidden = r.integer("hidden_size", minimum=1)
        n_heads = r.integer("num_attention_heads", minimum=1)
        n_kv_heads = r.integer("num_key_value_heads", minimum=1)
        intermediate = r.integer("intermediate_size", minimum=1)
        vocab = r.integer("vocab_size", minimum=1)
        max_position = r.integer("max_position_embeddings", minimum=1)
        rms_eps = r.number("rms_norm_eps")
        if rms_eps <= 0.0:
            raise ConfigError(f"{origin}: RMSNorm epsilon must be positive and finite, got {rms_eps}")

        if r.has("head_dim"):
            head_dim = r.integer("head_dim", minimum=1)
        elif hidden % n_heads == 0:
            head_dim = hidden // n_heads
        else:
            raise ConfigError(
                f"{origin}: 'head_dim' is missing and hidden_size {hidden} is not divisible by "
                f"{n_heads} attention heads")
        if head_dim % 2 != 0:
            raise ConfigError(f"{origin}: attention head dimension must be positive and even, got {head_dim}")
        if n_heads % n_kv_heads != 0:
            raise ConfigError(
                f"{origin}: {n_heads} query heads do not group evenly into {n_kv_heads} kv heads")

        rope_theta = cls._rope_theta(r, origin)

        # switches of the architecture family that this decoder does not implement
        if r.has("attention_bias") and r.boolean("attention_bias"):
            raise ConfigError(f"{origin}: attention_bias=true is not implemented (Qwen3 dense has no biases)")
        if r.has("mlp_bias") and r.boolean("mlp_bias"):
            raise ConfigError(f"{origin}: mlp_bias=true is not implemented (Qwen3 dense has no biases)")
        if r.has("hidden_act") and r.string("hidden_act") != "silu":
            raise ConfigError(f"{origin}: hidden_act {r.string('hidden_act')!r} is not implemented; only 'silu'")
        if r.has("use_sliding_window") and r.boolean("use_sliding_window"):
            raise ConfigError(f"{origin}: use_sliding_window=true is not implemented for Qwen3 dense")
        if r.has("layer_types"):
            kinds = r.raw("layer_types")
            if not isinstance(kinds, list) or len(kinds) != n_layers:
                raise ConfigError(f"{origin}: 'layer_types' must list {n_layers} layers")
            other = sorted({str(k) for k in kinds if k != "full_attention"})
            if other:
                raise ConfigError(f"{origin}: layer types {other} are not implemented; only 'full_attention'")
        if r.has("model_type") and r.string("model_type") != "qwen3":
            raise ConfigError(f"{origin}: model_type {r.string('model_type')!r} does not belong to {architecture}")

        tie = r.boolean("tie_word_embeddings", default=False)

        eos = data.get("eos_token_id")
        if eos is None:
            eos_ids: tuple = ()
        elif isinstance(eos, int) and not isinstance(eos, bool):
            eos_ids = (eos,)
        elif isinstance(eos, list) and all(isinstance(e, int) and not isinstance(e, bool) for e in eos):
            eos_ids = tuple(eos)
        else:
            raise ConfigError(f"{origin}: 'eos_token_id' must be an integer or a list of integers")
        for e in eos_ids:
            if not 0 <= e < vocab:
                raise ConfigError(f"{origin}: eos_token_id {e} is outside the vocabulary of {vocab}")

        return cls(architecture=architecture, n_layers=n_layers, hidden=hidden, n_heads=n_heads,
                   n_kv_heads=n_kv_heads, head_dim=head_dim, intermediate=intermediate, vocab=vocab,
                   rms_eps=rms_eps, rope_theta=rope_theta, max_position=max_position,
                   tie_word_embeddings=tie, eos_token_ids=eos_ids)

    @staticmethod
    def _rope_theta(r: ConfigReader, origin: str) -> float:
        """`rope_theta`, or the same number inside `rope_parameters`; any scaling is refused."""
        theta = None
        for key in ("rope_scaling", "rope_parameters"):
            if not r.has(key):
                continue
            block = r.raw(key)
            if not isinstance(block, dict):
                raise ConfigError(f"{origin}: {key!r} must be an object or null")
            kind = block.get("rope_type", block.get("type", "default"))
            if kind != "default":
                raise ConfigError(f"{origin}: rotation scaling {kind!r} ({key}) is not implemented; "
                                  "only plain rotation")
            if "rope_theta" in block:
                theta = ConfigReader(block, f"{origin}:{key}").number("rope_theta")
        if r.has("rope_theta"):
            theta = r.number("rope_theta")
        if theta is None:
            raise ConfigError(f"{origin}: required key 'rope_theta' is missing")
        if theta <= 0.0:
            raise ConfigError(f"{origin}: RoPE base must be positive and finite, got {theta}")
        return theta

    def to_dict(self) -> dict:
        """A config.json that reads back into this configuration."""
        out = {
            "architectures": [self.architecture],
            "model_type": "qwen3",
            "num_hidden_layers": self.n_layers,
            "hidden_size": self.hidden,
            "num_attention_heads": self.n_heads,
            "num_key_value_heads": self.n_kv_heads,
            "head_dim": self.head_dim,
            "intermediate_size": self.intermediate,
            "vocab_size": self.vocab,
            "rms_norm_eps": self.rms_eps,
            "rope_theta": self.rope_theta,
            "max_position_embeddings": self.max_position,
            "tie_word_embeddings": self.tie_word_embeddings,
            "hidden_act": "silu",
            "attention_bias": False,
        }
        if self.eos_token_ids:
            out["eos_token_id"] = list(self.eos_token_ids) if len(self.eos_token_ids) > 1 else self.eos_token_ids[0]
        return out
