"""Qwen3 dense: its typed configuration and configuration -> ``ModelSpec``.

Reference: ``jllm/model/qwen3.py:23-56`` (fields, keys and defaults of the configuration;
validation that the reference lacks is added: every size positive, heads divisible into
groups, an even head size), ``jllm/model/weights.py:113-155`` (which parts a layer has, their
tensor names, that all four norm kinds use ``rms_norm_eps``, rotary dim = head size, tied
head).  Every layer is the same here, but the spec lists them one by one: mixers and
feed-forwards are chosen per layer, and the schedule is a list.
"""
from __future__ import annotations

from dataclasses import dataclass, fields
from typing import Any, Mapping

from ..config.errors import ConfigError
from ..config.model import config_value, read_config_json
from ..config.registry import register_architecture
from ..parts.spec import LayerRun, LayerSpec, ModelSpec, PartSpec


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
        nq = config_value(c, "num_attention_heads", int)
        hidden = config_value(c, "hidden_size", int)
        if nq <= 0:
            raise ConfigError("num_attention_heads must be positive")
        cfg = cls(
            vocab_size=config_value(c, "vocab_size", int),
            hidden_size=hidden,
            intermediate_size=config_value(c, "intermediate_size", int),
            num_hidden_layers=config_value(c, "num_hidden_layers", int),
            num_heads=nq,
            num_kv_heads=config_value(c, "num_key_value_heads", int, nq, required=False),
            head_dim=config_value(c, "head_dim", int, hidden // nq, required=False),
            rms_norm_eps=config_value(c, "rms_norm_eps", float),
            rope_theta=config_value(c, "rope_theta", float, 1_000_000.0, required=False),
            max_position_embeddings=config_value(c, "max_position_embeddings", int),
            tie_word_embeddings=config_value(c, "tie_word_embeddings", bool, False, required=False),
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



def build_spec(cfg: Qwen3Config) -> ModelSpec:
    norm = PartSpec("rmsnorm", {"size": cfg.hidden_size, "eps": cfg.rms_norm_eps})
    mixer = PartSpec(
        "gqa_attention",
        {
            "hidden_size": cfg.hidden_size,
            "num_heads": cfg.num_heads,
            "num_kv_heads": cfg.num_kv_heads,
            "head_dim": cfg.head_dim,
            "qk_norm_eps": cfg.rms_norm_eps,
            "position": PartSpec("rotary", {"head_dim": cfg.head_dim, "theta": cfg.rope_theta}),
        },
    )
    ffn = PartSpec("gated_mlp", {"hidden_size": cfg.hidden_size, "intermediate_size": cfg.intermediate_size,
                                 "activation": "silu"})
    block = PartSpec("prenorm", {"norm": norm})
    layers = [
        LayerSpec(prefix=f"model.layers.{i}.", mixer=mixer, feed_forward=ffn, block=block,
                  mixer_prefix="self_attn.", feed_forward_prefix="mlp.")
        for i in range(cfg.num_hidden_layers)
    ]
    return ModelSpec(
        vocab_size=cfg.vocab_size,
        hidden_size=cfg.hidden_size,
        embedding=PartSpec("token_embedding", {"vocab_size": cfg.vocab_size, "hidden_size": cfg.hidden_size}),
        embedding_prefix="model.embed_tokens.",
        final_norm=norm,
        final_norm_prefix="model.norm.",
        head=PartSpec("linear_head", {"vocab_size": cfg.vocab_size, "hidden_size": cfg.hidden_size}),
        head_prefix="lm_head.",
        layers=layers,
        schedule=[LayerRun(i) for i in range(cfg.num_hidden_layers)],
        tie_head_to_embedding=cfg.tie_word_embeddings,
    )


register_architecture("Qwen3ForCausalLM", Qwen3Config.from_dict, build_spec)
