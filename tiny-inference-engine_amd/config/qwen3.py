"""Typed configuration of the Qwen3 dense decoder, read from its config.json keys.

Keys, defaults and rejections follow ``src/model/config.cpp:10-67`` of the
reference; every size and constant the model uses comes from here.
"""

from __future__ import annotations

import dataclasses
from typing import Any, Mapping

from ..errors import LoadError, UnsupportedError
from .base import ConfigReader


@dataclasses.dataclass(frozen=True)
class Qwen3Config:
    vocab_size: int
    hidden_size: int
    intermediate_size: int
    num_layers: int
    num_heads: int
    num_kv_heads: int
    head_dim: int
    max_position_embeddings: int
    rms_norm_eps: float
    rope_theta: float
    tie_word_embeddings: bool

    @property
    def q_dim(self) -> int:
        return self.num_heads * self.head_dim

    @property
    def kv_dim(self) -> int:
        return self.num_kv_heads * self.head_dim

    def validate(self) -> None:
        """Rejects inconsistent values (``config.cpp:14-28``)."""
        for field in ("vocab_size", "hidden_size", "intermediate_size", "num_layers", "num_heads",
                      "num_kv_heads", "head_dim", "max_position_embeddings"):
            value = getattr(self, field)
            if value <= 0:
                raise LoadError(f"config {field} must be positive, got {value}")
        if self.num_heads % self.num_kv_heads != 0:
            raise LoadError(f"num_heads {self.num_heads} is not a multiple of num_kv_heads {self.num_kv_heads}")
        if self.head_dim % 2 != 0:
            raise LoadError(f"head_dim {self.head_dim} must be even for rotary embeddings")
        if not (self.rms_norm_eps > 0.0) or not (self.rope_theta > 0.0):
            raise LoadError(
                f"rms_norm_eps ({self.rms_norm_eps}) and rope_theta ({self.rope_theta}) must be positive")

    @classmethod
    def from_json(cls, values: Mapping[str, Any]) -> "Qwen3Config":
        """Reads a HuggingFace Qwen3 config.json (``config.cpp:31-67``).

        Unknown keys are ignored. Options that would change the arithmetic and
        that this engine does not compute are refused rather than ignored:
        sliding-window attention, rope scaling, attention bias, and an
        activation other than SiLU (the reference fixes SiLU in code,
        ``src/backend/cpu/cpu_backend.cpp:195-207``).
        """
        r = ConfigReader(values)
        if r.boolean("use_sliding_window", False):
            raise UnsupportedError("use_sliding_window=true is not supported; Qwen3 here computes full attention")
        if r.has("rope_scaling"):
            raise UnsupportedError(f"rope_scaling {r.raw('rope_scaling')!r} is not supported")
        if r.boolean("attention_bias", False):
            raise UnsupportedError("attention_bias=true is not supported")
        act = r.string("hidden_act", "silu")
        if act != "silu":
            raise UnsupportedError(f"hidden_act '{act}' is not supported (supported: silu)")
        num_heads = r.integer("num_attention_heads")
        hidden = r.integer("hidden_size")
        if num_heads <= 0:
            raise LoadError(f"config num_heads must be positive, got {num_heads}")
        config = cls(
            vocab_size=r.integer("vocab_size"),
            hidden_size=hidden,
            intermediate_size=r.integer("intermediate_size"),
            num_layers=r.integer("num_hidden_layers"),
            num_heads=num_heads,
            num_kv_heads=r.integer("num_key_value_heads", num_heads),
            head_dim=r.integer("head_dim", hidden // num_heads),
            max_position_embeddings=r.integer("max_position_embeddings"),
            rms_norm_eps=r.number("rms_norm_eps"),
            rope_theta=r.number("rope_theta", 10000.0),
            tie_word_embeddings=r.boolean("tie_word_embeddings", False),
        )
        config.validate()
        return config

    def to_json(self) -> dict:
        """The config.json that reads back as this configuration."""
        return {
            "architectures": ["Qwen3ForCausalLM"],
            "model_type": "qwen3",
            "vocab_size": self.vocab_size,
            "hidden_size": self.hidden_size,
            "intermediate_size": self.intermediate_size,
            "num_hidden_layers": self.num_layers,
            "num_attention_heads": self.num_heads,
            "num_key_value_heads": self.num_kv_heads,
            "head_dim": self.head_dim,
            "max_position_embeddings": self.max_position_embeddings,
            "rms_norm_eps": self.rms_norm_eps,
            "rope_theta": self.rope_theta,
            "tie_word_embeddings": self.tie_word_embeddings,
            "hidden_act": "silu",
            "attention_bias": False,
            "use_sliding_window": False,
            "rope_scaling": None,
        }
