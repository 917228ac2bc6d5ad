"""Replays the same requests through bin/trace_run whole, with the last 32 tokens one by one,
in portions of changing size, and mixed with other requests in a pool so small that pages
are used again; in 32-bit and in bfloat16; every logit row is compared with the plain
whole-sequence implementation."""
import numpy as np
import pytest
import torch

from tests.plain import qwen3_plain as P
from tests.replay_util import Trace, compare, mixed, portions, run_trace, tail_one_by_one, whole
from tests.tiny import ALL_TINY

pytestmark = pytest.mark.gpu

LENGTHS = [70, 45, 100, 37, 64, 129]


@pytest.fixture(scope="module", params=ALL_TINY, ids=[t["name"] for t in ALL_TINY])
def tiny_model(request, tmp_path_factory):
    from jax_vllm_amd import write_random_model

    tiny = request.param
    folder = tmp_path_factory.mktemp(f"tiny{tiny['name']}")
    write_random_model(folder, tiny["config"], seed=tiny["seed"], std=tiny["std"], norm_std=tiny["norm_std"])
    cfg, w = P.read_config(folder), P.read_weights(folder)
    rng = np.random.default_rng(100 + tiny["seed"])
    requests = {f"r{i}": rng.integers(0, cfg["vocab_size"], size=n).tolist() for i, n in enumerate(LENGTHS)}
    expected = {name: P.forward(w, cfg, toks).numpy() for name, toks in requests.items()}
    return tiny, folder, requests, expected


def build_trace(requests, seed):
    rng = np.random.default_rng(seed)
    tr = Trace()
    for name, toks in requests.items():
        whole(tr, name + "#whole", toks)
    for name, toks in list(requests.items())[:3]:
        tail_one_by_one(tr, name + "#tail", toks, 32)
    portions(tr, "r2#cutA", requests["r2"], [7, 2, 13, 3, 2, 29, 16, 1])
    portions(tr, "r5#cutB", requests["r5"], [2, 2, 33, 15, 17, 2])
    portions(tr, "r0#cutC", requests["r0"], [16, 16, 16, 16, 6])
    peak = mixed(tr, {f"{n}#mix": t for n, t in requests.items()}, rng)
    return tr, peak


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_replay_every_cut_matches_plain(tiny_model, dtype, tmp_path):
    tiny, folder, requests, expected = tiny_model
    tr, peak = build_trace(requests, seed=7)
    # sized for the mixed part: four live requests, so released pages are taken again
    max_tokens = max(peak, 192)
    got = run_trace(folder, dtype, tr, max_tokens, tmp_path / "out", block_size=tiny["page_size"])
    scale = max(float(np.abs(e).max()) for e in expected.values())
    worst = {"err": 0.0, "cos": 1.0}

    def check(name, pos, g, w):
        err = float(np.abs(g - w).max())
        worst["err"] = max(worst["err"], err)
        if dtype == "float32":
            assert err <= 2e-5 * max(scale, 1.0) + 1e-5, f"{name} position {pos}: max error {err}"
        else:
            cos = float(np.dot(g, w) / (np.linalg.norm(g) * np.linalg.norm(w) + 1e-30))
            worst["cos"] = min(worst["cos"], cos)
            assert err <= 0.03 * scale + 1e-3, f"{name} position {pos}: max error {err} (scale {scale})"
            assert cos >= 0.999, f"{name} position {pos}: cosine {cos}"

    n = compare(tr, got, expected, check)
    assert n > 1000
    print(f"\n[{tiny['name']} {dtype}] rows {n}, scale {scale:.3f}, worst error {worst['err']:.3e}, worst cosine {worst['cos']:.6f}")
