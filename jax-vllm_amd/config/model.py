"""Typed model configuration read from the architecture's own ``config.json`` keys.

Reference: ``jllm/model/qwen3.py:23-56`` (fields, keys and defaults of ``Qwen3Config``).
Validation that the reference lacks is added here: every size positive, heads
divisible into groups, a head size the kernels accept.
"""
from __future__ import annotations

import json
from dataclasses import dataclass, fields
from pathlib import Path
from typing import Any, Mapping

from .errors import ConfigError


def read_config_json(path) -> dict:
    """``config.json`` of a model folder (or the file itself) as a dict."""
    p = Path(path)
    if p.is_dir():
        p = p / "config.json"
    if not p.exists():
        raise ConfigError(f"no config.json at {p}")
    try:
        data = json.loads(p.read_text())
    except json.JSONDecodeError as e:
        raise ConfigError(f"{p} is not valid JSON: {e}") from e
    if not isinstance(data, dict):
        raise ConfigError(f"{p} must hold a JSON object")
    return data


def _get(c: Mapping[str, Any], key: str, typ, default=None, required=True):
    if key not in c or c[key] is None:
        if required:
            raise ConfigError(f"config.json lacks the required key {key!r}")
        return default
    v = c[key]
    if typ is float and isinstance(v, int) and not isinstance(v, bool):
        v = float(v)
    if typ is int and isinstance(v, bool) or not isinstance(v, typ):
        raise ConfigError(f"config.json key {key!r} must be {typ.__name__}, got {v!r}")
    return v


@dataclass(frozen=True)
class Qwen3Config:
    """Qwen3 dense decoder (``jllm/model/qwen3.py:23-35``)."""

    vocab_size: int
    hidden_size: int
    intermediate_size: int
    num_hidden_layers: int
    num_heads: int
    num_kv_heads: int
    head_dim: int
    rms_norm_eps: float
    rope_theta: float
    max_position_embeddings: int
    tie_word_embeddings: bool

    @classmethod
    def from_dict(cls, c: Mapping[str, Any]) -> "Qwen3Config":
        """Keys and defaults as in ``jllm/model/qwen3.py:43-55``: kv heads default to the
        q heads, the head size to hidden / heads, rope_theta to 1e6, untied head."""
        nq = _get(c, "num_attention_heads", int)
        hidden = _get(c, "hidden_size", int)
        if nq <= 0:
            raise ConfigError("num_attention_heads must be positive")
        cfg = cls(
            vocab_size=_get(c, "vocab_size", int),
            hidden_size=hidden,
            intermediate_size=_get(c, "intermediate_size", int),
            num_hidden_layers=_get(c, "num_hidden_layers", int),
            num_heads=nq,
            num_kv_heads=_get(c, "num_key_value_heads", int, nq, required=False),
            head_dim=_get(c, "head_dim", int, hidden // nq, required=False),
            rms_norm_eps=_get(c, "rms_norm_eps", float),
            rope_theta=_get(c, "rope_theta", float, 1_000_000.0, required=False),
            max_position_embeddings=_get(c, "max_position_embeddings", int),
            tie_word_embeddings=_get(c, "tie_word_embeddings", bool, False, required=False),
        )
        # Options of the checkpoint format that the reference's Qwen3 does not compute:
        # accepting them silently would give wrong results.
        if c.get("use_sliding_window"):
            raise ConfigError("use_sliding_window=true is not part of this architecture (full causal attention)")
        if c.get("rope_scaling") not in (None, {}):
            raise ConfigError("rope_scaling is not part of this architecture")
        if c.get("attention_bias"):
            raise ConfigError("attention_bias=true is not part of this architecture (no biases)")
        if c.get("hidden_act", "silu") != "silu":
            raise ConfigError(f"hidden_act must be 'silu', got {c.get('hidden_act')!r}")
        cfg.validate()
        return cfg

    @classmethod
    def from_folder(cls, path) -> "Qwen3Config":
        return cls.from_dict(read_config_json(path))

    def validate(self) -> None:
        for f in fields(self):
            v = getattr(self, f.name)
            if f.type in ("int", int) and v <= 0:
                raise ConfigError(f"{f.name} must be positive, got {v}")
        if self.num_heads % self.num_kv_heads != 0:
            raise ConfigError(
                f"num_attention_heads ({self.num_heads}) must be a multiple of num_key_value_heads ({self.num_kv_heads})"
            )
        if self.head_dim % 2 != 0:
            raise ConfigError(f"head_dim ({self.head_dim}) must be even for the rotary pairing")
        if not (self.rms_norm_eps >= 0.0):
            raise ConfigError("rms_norm_eps must be non-negative")
        if not (self.rope_theta > 0.0):
            raise ConfigError("rope_theta must be positive")

    def to_dict(self) -> dict:
        """The ``config.json`` form (used when a random-weights folder is written)."""
        return {
            "architectures": ["Qwen3ForCausalLM"],
            "model_type": "qwen3",
            "vocab_size": self.vocab_size,
            "hidden_size": self.hidden_size,
            "intermediate_size": self.intermediate_size,
            "num_hidden_layers": self.num_hidden_layers,
            "num_attention_heads": self.num_heads,
            "num_key_value_heads": self.num_kv_heads,
            "head_dim": self.head_dim,
            "rms_norm_eps": self.rms_norm_eps,
            "rope_theta": self.rope_theta,
            "max_position_embeddings": self.max_position_embeddings,
            "tie_word_embeddings": self.tie_word_embeddings,
            "hidden_act": "silu",
        }
