"""Helpers of the GPU tests: tiny model folders, engines on them, and the comparison rule."""
import numpy as np
import torch

from tests.plain import qwen3_plain as P


def make_folder(tiny, tmp_path):
    from jax_vllm_amd import write_random_model

    return write_random_model(tmp_path, tiny["config"], seed=tiny["seed"], std=tiny["std"], norm_std=tiny["norm_std"])


def plain_of(folder):
    return P.read_config(folder), P.read_weights(folder)


def make_core(folder, dtype, page_size, pages=64, seqs=4, graphs=False, prefix=False, model=None):
    from jax_vllm_amd.config import EngineConfig
    from jax_vllm_amd.engine.core import EngineCore
    from jax_vllm_amd.weights import load_model

    if model is None:
        model, _ = load_model(folder, dtype, "cuda")
    cfg = EngineConfig(dtype=dtype, block_size=page_size, num_blocks=pages + 1, max_num_seqs=seqs,
                       max_model_len=pages * page_size, max_num_batched_tokens=4096, enable_prefix_cache=prefix,
                       use_hip_graphs=graphs)
    return EngineCore(model, cfg)


def check_logits(dtype, got, want, scale=None, what=""):
    """float32: agreement to float rounding of a deep sum.  bfloat16: error below 3% of the
    largest logit and cosine above 0.999 (the reference's own bf16 bar is cosine > 0.998 and
    equal argmax, tests/test_parity.py:26-29 there)."""
    got = np.asarray(got, dtype=np.float64)
    want = np.asarray(want, dtype=np.float64)
    assert got.shape == want.shape, f"{what}: shapes {got.shape} and {want.shape}"
    scale = float(np.abs(want).max()) if scale is None else scale
    err = float(np.abs(got - want).max())
    if dtype in ("float32", "fp32"):
        assert err <= 2e-5 * max(scale, 1.0) + 1e-5, f"{what}: max error {err} (scale {scale})"
    else:
        assert err <= 0.03 * scale + 1e-3, f"{what}: max error {err} (scale {scale})"
        g, w = got.reshape(-1, got.shape[-1]), want.reshape(-1, want.shape[-1])
        cos = (g * w).sum(-1) / (np.linalg.norm(g, axis=-1) * np.linalg.norm(w, axis=-1) + 1e-30)
        assert cos.min() >= 0.999, f"{what}: cosine {cos.min()}"
    return err


def check_tokens_follow(dtype, cfg, w, prompt, tokens, scale_margin=0.04):
    """Every generated token is an argmax of the plain logits given everything before it; in
    bfloat16 a token within a small margin of the maximum is accepted (ties broken by rounding)."""
    seq = list(prompt)
    for i, t in enumerate(tokens):
        logits = P.forward(w, cfg, seq)[-1]
        if dtype in ("float32", "fp32"):
            assert int(torch.argmax(logits)) == t, f"token {i}: engine {t}, plain {int(torch.argmax(logits))}"
        else:
            margin = float(logits.max() - logits[t])
            assert margin <= scale_margin * float(logits.abs().max()), f"token {i}: engine {t} is {margin} below the maximum"
        seq.append(t)
