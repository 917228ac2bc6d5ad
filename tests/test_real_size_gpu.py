"""The layer sizes of real models (Qwen3-8B: hidden 4096, 32/8 heads of 128, feed-forward
12288, vocabulary 151936; the 14B sizes: hidden 5120, 40/8 heads, feed-forward 17408; the 32B
sizes: hidden 5120, 64/8 heads, so that heads * head size = 8192 is not the width, feed-forward
25600) with two layers of random weights: the 32-bit path and the bfloat16
path against the plain implementation, whole, token by token, in portions and mixed.  These are
the sizes at which the kernels' wide paths run (16-byte norm loads, the streaming matrix
product's real shapes, a vocabulary that is no power of two, the 128-wide MFMA attention)."""
import numpy as np
import pytest
import torch

from tests.gpu_util import check_logits, make_core
from tests.plain import qwen3_plain as P

pytestmark = pytest.mark.gpu

CONFIG = dict(architectures=["Qwen3ForCausalLM"], num_hidden_layers=2, hidden_size=4096, num_attention_heads=32,
              num_key_value_heads=8, head_dim=128, intermediate_size=12288, vocab_size=151936, rope_theta=1000000.0,
              rms_norm_eps=1e-6, tie_word_embeddings=False, max_position_embeddings=40960)
# the next size up: 5 query heads per kv head, a width of 5120 (inner sizes that are no multiple of
# 4096: other organisations of the streaming products), a feed-forward of 17408
CONFIG_14B = dict(CONFIG, hidden_size=5120, num_attention_heads=40, intermediate_size=17408)
# 8 query heads per kv head; the attention's output is wider than the model (8192 against 5120), the
# feed-forward's inner size is beyond what one block keeps of x: further branches of the products' plans
CONFIG_32B = dict(CONFIG, hidden_size=5120, num_attention_heads=64, intermediate_size=25600)


@pytest.fixture(scope="module", params=[CONFIG, CONFIG_14B, CONFIG_32B], ids=["8b", "14b", "32b"])
def big(request):
    CONFIG = request.param
    from jax_vllm_amd.config import resolve
    from jax_vllm_amd.parts import DecoderModel
    from jax_vllm_amd.weights.random_init import _draw

    arch, cfg, _ = resolve(CONFIG)
    spec = arch.build_spec(cfg)
    names = DecoderModel(spec).tensor_specs()
    dev = {n: _draw(ts, 0, n, 0.02, 0.02, device="cuda").to(torch.bfloat16) for n, ts in names.items()}
    plain_w = {n: t.float().cpu() for n, t in dev.items()}
    plain_cfg = dict(vocab_size=cfg.vocab_size, hidden_size=cfg.hidden_size, intermediate_size=cfg.intermediate_size,
                     num_hidden_layers=cfg.num_hidden_layers, num_heads=cfg.num_heads, num_kv_heads=cfg.num_kv_heads,
                     head_dim=cfg.head_dim, rms_norm_eps=cfg.rms_norm_eps, rope_theta=cfg.rope_theta,
                     tie_word_embeddings=cfg.tie_word_embeddings)
    rng = np.random.default_rng(0)
    reqs = {f"r{i}": rng.integers(0, cfg.vocab_size, size=n).tolist() for i, n in enumerate((64, 150, 300, 97))}
    torch.set_num_threads(16)
    want = {r: P.forward(plain_w, plain_cfg, t).numpy() for r, t in reqs.items()}

    def model(dtype):
        from jax_vllm_amd.weights.loader import target_dtype

        compute = torch.float32 if dtype == "float32" else torch.bfloat16
        m = DecoderModel(spec)
        m.bind({n: dev[n].to(target_dtype(names[n].role, compute)).contiguous() for n in names}, compute)
        return m

    return model, reqs, want


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_real_layer_sizes_every_cut(big, dtype):
    from jax_vllm_amd.engine.entries import StepEntry

    model, reqs, want = big
    core = make_core(None, dtype, 16, pages=48, seqs=4, model=model(dtype), graphs=(dtype == "bfloat16"))
    scale = max(float(np.abs(w).max()) for w in want.values())

    def run(entries):
        out = core.run([StepEntry(r, t, range(len(t))) for r, t in entries]).cpu().numpy()
        res, at = [], 0
        for r, t in entries:
            res.append(out[at:at + len(t)])
            at += len(t)
        return res

    # whole, then most of it in one step and the last 32 tokens one by one
    for r, toks in reqs.items():
        core.start_request(r)
        check_logits(dtype, run([(r, toks)])[0], want[r], scale, f"{r} whole")
        core.finish_request(r)
    r, toks = "r1", reqs["r1"]
    core.start_request(r)
    got = run([(r, toks[:-32])])
    for i in range(len(toks) - 32, len(toks)):
        got += run([(r, toks[i:i + 1])])
    check_logits(dtype, np.concatenate(got), want[r], scale, f"{r} tail one by one")
    core.finish_request(r)
    # portions of changing size beside single tokens of other requests, pages taken again
    fed = {r: 0 for r in reqs}
    got = {r: [] for r in reqs}
    for r in reqs:
        core.start_request(r)
    # (the third step has 40 tokens in all: the matrix products for 17..64 rows)
    sizes = {"r0": [7, 2, 9, 24, 22], "r1": [64, 2, 11, 59, 14], "r2": [100, 3, 13, 137, 47], "r3": [1, 1, 7, 1, 87]}
    for step in range(5):
        entries = [(r, reqs[r][fed[r]:fed[r] + sizes[r][step]]) for r in reqs]
        for (r, t), o in zip(entries, run(entries)):
            got[r].append(o)
            fed[r] += len(t)
    for r in reqs:
        assert fed[r] == len(reqs[r])
        check_logits(dtype, np.concatenate(got[r]), want[r], scale, f"{r} mixed")
        core.finish_request(r)
    core.cache.check_invariants()
