"""Tiny Qwen3 configurations of the test-suite.  They differ in every size and option:
layer count, width, head counts and group ratio, head size, feed-forward width,
vocabulary, rope_theta, eps, tied or untied head, page size, weight scale."""
import torch


def _cfg(**kw):
    base = dict(architectures=["Qwen3ForCausalLM"], model_type="qwen3", hidden_act="silu",
                max_position_embeddings=4096, torch_dtype="bfloat16")
    base.update(kw)
    return base


TINY_A = dict(
    name="A", seed=0, std=0.02, norm_std=0.02, page_size=8,
    config=_cfg(num_hidden_layers=2, hidden_size=64, num_attention_heads=4, num_key_value_heads=2,
                head_dim=16, intermediate_size=128, vocab_size=256, rope_theta=10000.0,
                rms_norm_eps=1e-6, tie_word_embeddings=True),
)
TINY_B = dict(
    name="B", seed=1, std=0.05, norm_std=0.1, page_size=16,
    config=_cfg(num_hidden_layers=3, hidden_size=96, num_attention_heads=6, num_key_value_heads=2,
                head_dim=32, intermediate_size=224, vocab_size=512, rope_theta=1000000.0,
                rms_norm_eps=1e-5, tie_word_embeddings=False),
)
# no size a power of two; one head per group; a head size that is a multiple of 16 only
TINY_C = dict(
    name="C", seed=2, std=0.08, norm_std=0.2, page_size=32,
    config=_cfg(num_hidden_layers=2, hidden_size=80, num_attention_heads=5, num_key_value_heads=5,
                head_dim=48, intermediate_size=176, vocab_size=777, rope_theta=500000.0,
                rms_norm_eps=1e-4, tie_word_embeddings=False),
)
ALL_TINY = [TINY_A, TINY_B, TINY_C]


def tensor_shapes(config: dict) -> dict:
    """HF tensor names and shapes of a Qwen3 checkpoint (reference: jllm/model/weights.py:118-152)."""
    h, i, v = config["hidden_size"], config["intermediate_size"], config["vocab_size"]
    nq, nkv, d = config["num_attention_heads"], config["num_key_value_heads"], config["head_dim"]
    s = {"model.embed_tokens.weight": (v, h), "model.norm.weight": (h,)}
    if not config["tie_word_embeddings"]:
        s["lm_head.weight"] = (v, h)
    for l in range(config["num_hidden_layers"]):
        p = f"model.layers.{l}"
        s[f"{p}.input_layernorm.weight"] = (h,)
        s[f"{p}.post_attention_layernorm.weight"] = (h,)
        s[f"{p}.self_attn.q_proj.weight"] = (nq * d, h)
        s[f"{p}.self_attn.k_proj.weight"] = (nkv * d, h)
        s[f"{p}.self_attn.v_proj.weight"] = (nkv * d, h)
        s[f"{p}.self_attn.o_proj.weight"] = (h, nq * d)
        s[f"{p}.self_attn.q_norm.weight"] = (d,)
        s[f"{p}.self_attn.k_norm.weight"] = (d,)
        s[f"{p}.mlp.gate_proj.weight"] = (i, h)
        s[f"{p}.mlp.up_proj.weight"] = (i, h)
        s[f"{p}.mlp.down_proj.weight"] = (h, i)
    return s


def make_weights_dict(tiny: dict, dtype=torch.float32) -> dict:
    """Seeded weights for the plain implementation alone (CPU tests): matrices N(0, std),
    norm weights 1 + N(0, norm_std), rounded through bfloat16 like a stored checkpoint."""
    g = torch.Generator().manual_seed(1000 + tiny["seed"])
    out = {}
    for name, shape in tensor_shapes(tiny["config"]).items():
        if len(shape) == 1:
            t = 1.0 + tiny["norm_std"] * torch.randn(shape, generator=g)
        else:
            t = tiny["std"] * torch.randn(shape, generator=g)
        out[name] = t.to(torch.bfloat16).to(dtype)
    return out
