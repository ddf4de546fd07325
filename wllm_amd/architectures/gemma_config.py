"""Typed configuration of Gemma 1 (`GemmaForCausalLM`), read from its config.json keys.

Keys and defaults follow the reference's `ModelConfig.from_json`
(src/wllm/models/config.py:38-71): `vocab_size`, `hidden_size`,
`intermediate_size`, `num_hidden_layers`, `num_attention_heads` are required;
`num_key_value_heads` defaults to the number of heads, `rms_norm_eps` to 1e-6,
`rope_theta` (also under `rope_parameters`) to 10000.0,
`max_position_embeddings` to 4096, `head_dim` to hidden_size // heads when the
key is absent (config.py:32-36), `attention_bias` to False for this model type
(config.py:54-56).  Two departures: `tie_word_embeddings` defaults to True, as
Gemma 1 checkpoints are tied (the reference defaults to False, config.py:68),
and `max_position_embeddings` is enforced as a limit on a request's length
(the reference parses it and never uses it).  Gelu-tanh, the sqrt(hidden)
embedding factor, the half-split rotation and the (1 + w) norm are properties
of the architecture (src/wllm/models/gemma.py:41-62,158-162), not keys.
"""
from __future__ import annotations

from dataclasses import asdict, dataclass

from wllm_amd.config.registry import ConfigError

_REQUIRED = ("vocab_size", "hidden_size", "intermediate_size", "num_hidden_layers", "num_attention_heads")


@dataclass(frozen=True)
class GemmaConfig:
    vocab_size: int
    hidden_size: int
    intermediate_size: int
    num_hidden_layers: int
    num_attention_heads: int
    num_key_value_heads: int
    head_dim: int
    rms_norm_eps: float = 1e-6
    rope_theta: float = 10000.0
    max_position_embeddings: int = 4096
    tie_word_embeddings: bool = True
    attention_bias: bool = False

    def __post_init__(self):
        for key in _REQUIRED + ("num_key_value_heads", "head_dim", "max_position_embeddings"):
            v = getattr(self, key)
            if isinstance(v, bool) or not isinstance(v, int) or v <= 0:
                raise ConfigError(f"{key} must be a positive integer, got {v!r}")
        if self.num_attention_heads % self.num_key_value_heads != 0:
            raise ConfigError(
                f"num_attention_heads ({self.num_attention_heads}) must be a multiple of "
                f"num_key_value_heads ({self.num_key_value_heads})")
        if self.head_dim % 2 != 0:
            raise ConfigError(f"head_dim must be even for the half-split rotation, got {self.head_dim}")
        if not (isinstance(self.rms_norm_eps, float) and self.rms_norm_eps >= 0.0):
            raise ConfigError(f"rms_norm_eps must be a non-negative number, got {self.rms_norm_eps!r}")
        if not (isinstance(self.rope_theta, float) and self.rope_theta > 0.0):
            raise ConfigError(f"rope_theta must be a positive number, got {self.rope_theta!r}")

    @classmethod
    def from_dict(cls, raw: dict) -> "GemmaConfig":
        missing = [k for k in _REQUIRED if k not in raw]
        if missing:
            raise ConfigError(f"config.json lacks required key(s): {', '.join(missing)}")
        rope_theta = raw.get("rope_theta")
        if rope_theta is None:
            rope_theta = (raw.get("rope_parameters") or {}).get("rope_theta", 10000.0)
        heads = raw["num_attention_heads"]
        head_dim = raw.get("head_dim")
        if head_dim is None:
            if not isinstance(heads, int) or heads <= 0 or raw["hidden_size"] % heads != 0:
                raise ConfigError("head_dim is absent and hidden_size is not a multiple of num_attention_heads")
            head_dim = raw["hidden_size"] // heads
        kv_heads = raw.get("num_key_value_heads")
        if kv_heads is None:
            kv_heads = heads
        try:
            return cls(
                vocab_size=raw["vocab_size"],
                hidden_size=raw["hidden_size"],
                intermediate_size=raw["intermediate_size"],
                num_hidden_layers=raw["num_hidden_layers"],
                num_attention_heads=heads,
                num_key_value_heads=kv_heads,
                head_dim=head_dim,
                rms_norm_eps=float(raw.get("rms_norm_eps", 1e-6)),
                rope_theta=float(rope_theta),
                max_position_embeddings=raw.get("max_position_embeddings", 4096),
                tie_word_embeddings=bool(raw.get("tie_word_embeddings", True)),
                attention_bias=bool(raw.get("attention_bias") or False),
            )
        except (TypeError, ValueError) as e:
            if isinstance(e, ConfigError):
                raise
            raise ConfigError(f"config.json holds a value of the wrong type: {e}") from e

    def to_dict(self) -> dict:
        """The config.json of this configuration."""
        d = asdict(self)
        d["architectures"] = ["GemmaForCausalLM"]
        d["model_type"] = "gemma"
        return d
