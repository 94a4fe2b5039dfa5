"""Typed model configuration, read from the architecture's own config.json keys.

Every size and constant of the model comes from here; nothing downstream carries a
number of its own.  Field meanings and the rejected options follow the reference
(atomserve/config.py:15-65).
"""

from dataclasses import dataclass


class ConfigError(ValueError):
    """config.json names something this engine does not compute."""


def _require(raw: dict, keys: list[str]) -> None:
    missing = [k for k in keys if k not in raw]
    if missing:
        raise ConfigError(f"config.json lacks required key(s): {', '.join(missing)}")


@dataclass(frozen=True)
class Qwen3Config:
    """Shape and numerics of a Qwen3 dense decoder (reference atomserve/config.py:19-29)."""

    vocab_size: int  # rows of the embedding and of the head
    hidden_size: int  # width of the residual stream
    intermediate_size: int  # width inside the gated feed-forward
    num_layers: int  # decoder layers
    num_heads: int  # query heads
    num_kv_heads: int  # key/value heads; fewer than query heads means grouped queries
    head_dim: int  # width of one head; heads * head_dim need not equal hidden_size
    rms_norm_eps: float  # epsilon of every RMSNorm, the per-head q/k norms included
    rope_theta: float  # base of the rotary frequencies
    tie_word_embeddings: bool  # the head is the embedding table
    max_position_embeddings: int  # longest context the model was trained for

    architecture = "Qwen3ForCausalLM"

    @classmethod
    def from_dict(cls, raw: dict) -> "Qwen3Config":
        """Validate a parsed config.json; anything that would change the math is refused
        rather than ignored (reference atomserve/config.py:31-60)."""
        for key, why in (
            ("attention_bias", "projection biases are not computed"),
            ("rope_scaling", "scaled rotary frequencies are not computed"),
            ("use_sliding_window", "sliding-window attention is not part of this architecture here"),
        ):
            if raw.get(key):
                raise ConfigError(f"{key}={raw[key]!r} is not supported: {why}")
        if raw.get("hidden_act", "silu") != "silu":
            raise ConfigError(f"hidden_act={raw['hidden_act']!r} is not supported (only 'silu')")
        _require(
            raw,
            ["vocab_size", "hidden_size", "intermediate_size", "num_hidden_layers",
             "num_attention_heads", "num_key_value_heads", "rms_norm_eps", "rope_theta",
             "max_position_embeddings"],
        )  # fmt: skip
        heads = int(raw["num_attention_heads"])
        cfg = cls(
            vocab_size=int(raw["vocab_size"]),
            hidden_size=int(raw["hidden_size"]),
            intermediate_size=int(raw["intermediate_size"]),
            num_layers=int(raw["num_hidden_layers"]),
            num_heads=heads,
            num_kv_heads=int(raw["num_key_value_heads"]),
            head_dim=int(raw.get("head_dim") or int(raw["hidden_size"]) // heads),
            rms_norm_eps=float(raw["rms_norm_eps"]),
            rope_theta=float(raw["rope_theta"]),
            tie_word_embeddings=bool(raw.get("tie_word_embeddings", False)),
            max_position_embeddings=int(raw["max_position_embeddings"]),
        )
        cfg.validate()
        return cfg

    def validate(self) -> None:
        for name in ("vocab_size", "hidden_size", "intermediate_size", "num_layers", "num_heads",
                     "num_kv_heads", "head_dim", "max_position_embeddings"):  # fmt: skip
            if getattr(self, name) < 1:
                raise ConfigError(f"{name} must be positive, got {getattr(self, name)}")
        if self.num_heads % self.num_kv_heads:
            raise ConfigError(
                f"num_attention_heads {self.num_heads} is not a multiple of "
                f"num_key_value_heads {self.num_kv_heads}"
            )
        if self.head_dim % 2:
            raise ConfigError(f"head_dim {self.head_dim} must be even (rotary pairs)")
        if not self.rms_norm_eps > 0 or not self.rope_theta > 0:
            raise ConfigError("rms_norm_eps and rope_theta must be positive")

    def to_dict(self) -> dict:
        """The config.json that `from_dict` reads back to this object."""
        return {
            "architectures": [self.architecture],
            "model_type": "qwen3",
            "vocab_size": self.vocab_size,
            "hidden_size": self.hidden_size,
            "intermediate_size": self.intermediate_size,
            "num_hidden_layers": self.num_layers,
            "num_attention_heads": self.num_heads,
            "num_key_value_heads": self.num_kv_heads,
            "head_dim": self.head_dim,
            "hidden_act": "silu",
            "rms_norm_eps": self.rms_norm_eps,
            "rope_theta": self.rope_theta,
            "tie_word_embeddings": self.tie_word_embeddings,
            "max_position_embeddings": self.max_position_embeddings,
            "attention_bias": False,
            "torch_dtype": "bfloat16",
        }
