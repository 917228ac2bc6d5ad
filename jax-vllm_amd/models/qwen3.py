"""Qwen3 dense: configuration -> ``ModelSpec``.

Reference: ``jllm/model/weights.py:113-155`` (which parts a layer has, their tensor names,
that all four norm kinds use ``rms_norm_eps``, rotary dim = head size, tied head) and
``jllm/model/qwen3.py``.  Every layer is the same here, but the spec lists them one by
one: mixers and feed-forwards are chosen per layer, and the schedule is a list.
"""
from __future__ import annotations

from ..config.model import Qwen3Config
from ..config.registry import register_architecture
from ..parts.spec import LayerRun, LayerSpec, ModelSpec, PartSpec


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
    ffn = PartSpec("gated_mlp", {"hidden_size": cfg.hidden_size, "intermediate_size": cfg.intermediate_size})
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
