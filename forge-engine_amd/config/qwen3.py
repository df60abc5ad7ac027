"""Configuration of the Qwen3 dense decoder, from its config.json keys.

The reference reads the same thirteen keys (src/forge_engine/qwen3.py:18-62)
and then pins every one to a single checkpoint (64-88); here any consistent
set of sizes is accepted.  The three rejections of the reference are kept:
another ``model_type``, another ``hidden_act``, a sliding window (40-45).
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Any, ClassVar

from .model import ConfigError, KeyReader, ModelConfig


@dataclass(frozen=True)
class Qwen3Config(ModelConfig):
    vocab_size: int
    hidden_size: int
    intermediate_size: int
    num_hidden_layers: int
    num_attention_heads: int
    num_key_value_heads: int
    head_dim: int
    max_position_embeddings: int
    rms_norm_eps: float
    rope_theta: float
    eos_token_id: int | tuple[int, ...] | None = None
    tie_word_embeddings: bool = False
    attention_bias: bool = False

    architecture: ClassVar[str] = "Qwen3ForCausalLM"

    def __post_init__(self) -> None:
        if self.num_attention_heads % self.num_key_value_heads:
            raise ConfigError(
                f"num_attention_heads ({self.num_attention_heads}) must be a multiple of "
                f"num_key_value_heads ({self.num_key_value_heads})")
        if self.head_dim % 2:
            raise ConfigError(f"head_dim ({self.head_dim}) must be even for rotary positions")

    @property
    def q_size(self) -> int:
        return self.num_attention_heads * self.head_dim

    @property
    def kv_size(self) -> int:
        return self.num_key_value_heads * self.head_dim

    @property
    def groups(self) -> int:
        return self.num_attention_heads // self.num_key_value_heads

    @property
    def eos_token_ids(self) -> frozenset[int]:
        if self.eos_token_id is None:
            return frozenset()
        if isinstance(self.eos_token_id, int):
            return frozenset({self.eos_token_id})
        return frozenset(self.eos_token_id)

    @classmethod
    def from_dict(cls, raw: dict[str, Any]) -> "Qwen3Config":
        if raw.get("model_type", "qwen3") != "qwen3":
            raise ConfigError(f"model_type must be 'qwen3', got {raw.get('model_type')!r}")
        if raw.get("hidden_act", "silu") != "silu":
            raise ConfigError(f"hidden_act must be 'silu', got {raw.get('hidden_act')!r}")
        if raw.get("sliding_window") is not None and raw.get("use_sliding_window", True):
            raise ConfigError("sliding-window attention is not part of Qwen3 dense")
        if raw.get("rope_scaling") is not None:
            raise ConfigError("rope_scaling is not supported")
        read = KeyReader(raw)
        hidden = read.integer("hidden_size")
        heads = read.integer("num_attention_heads")
        default_head_dim = hidden // heads if hidden % heads == 0 else None
        eos = raw.get("eos_token_id")
        if isinstance(eos, list):
            eos = tuple(int(v) for v in eos)
        elif eos is not None:
            if isinstance(eos, bool) or not isinstance(eos, int):
                raise ConfigError(f"'eos_token_id' must be an integer or a list, got {eos!r}")
        return cls(
            vocab_size=read.integer("vocab_size"),
            hidden_size=hidden,
            intermediate_size=read.integer("intermediate_size"),
            num_hidden_layers=read.integer("num_hidden_layers"),
            num_attention_heads=heads,
            num_key_value_heads=read.integer("num_key_value_heads", heads),
            head_dim=read.integer("head_dim", default_head_dim),
            max_position_embeddings=read.integer("max_position_embeddings"),
            rms_norm_eps=read.number("rms_norm_eps"),
            rope_theta=read.number("rope_theta"),
            eos_token_id=eos,
            tie_word_embeddings=read.boolean("tie_word_embeddings", False),
            attention_bias=read.boolean("attention_bias", False),
        )

    def to_dict(self) -> dict[str, Any]:
        data = super().to_dict()
        if isinstance(data["eos_token_id"], tuple):
            data["eos_token_id"] = list(data["eos_token_id"])
        data.update(model_type="qwen3", hidden_act="silu", sliding_window=None)
        return data
