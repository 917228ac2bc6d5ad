"""Pins the plain implementation by what fixes it beside the reference's text:
library routines it must reduce to, invariants, and the reference's own vectors."""
import math

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from tests.plain import qwen3_plain as P
from tests.tiny import TINY_A, TINY_B, TINY_C, make_weights_dict


def test_rms_norm_is_library_rms_norm():
    g = torch.Generator().manual_seed(0)
    x = torch.randn(5, 7, 24, generator=g)
    w = 1 + 0.1 * torch.randn(24, generator=g)
    ref = F.rms_norm(x, (24,), w, 1e-5)
    torch.testing.assert_close(P.rms_norm(w, 1e-5, x), ref, rtol=1e-6, atol=1e-6)


def test_rms_norm_invariants():
    g = torch.Generator().manual_seed(1)
    x = torch.randn(3, 40, generator=g)
    y = P.rms_norm(torch.ones(40), 0.0, x)
    torch.testing.assert_close((y * y).mean(-1), torch.ones(3), rtol=1e-5, atol=1e-5)
    # scale invariance (a norm applied after the weight, or a mean instead of a mean square, breaks it)
    torch.testing.assert_close(P.rms_norm(torch.ones(40), 0.0, 7.5 * x), y, rtol=1e-5, atol=1e-5)
    # eps sits inside the square root, next to the mean square
    z = P.rms_norm(torch.ones(40), 3.0, x)
    torch.testing.assert_close(z, x / torch.sqrt((x * x).mean(-1, keepdim=True) + 3.0))


def test_rope_position_zero_is_identity_and_pairs_are_rotated():
    d = 16
    g = torch.Generator().manual_seed(2)
    x = torch.randn(3, 5, d, generator=g)
    pos = torch.tensor([0, 1, 7, 100, 4095])
    cos, sin = P.rope_cos_sin(d, 10000.0, pos, torch.float32)
    y = P.apply_rope(x, cos, sin)
    torch.testing.assert_close(y[:, 0], x[:, 0])
    # element i pairs with i + d/2: each such pair keeps its length (pairing (2i, 2i+1) fails this)
    n_in = x[..., : d // 2] ** 2 + x[..., d // 2 :] ** 2
    n_out = y[..., : d // 2] ** 2 + y[..., d // 2 :] ** 2
    torch.testing.assert_close(n_in, n_out, rtol=1e-4, atol=1e-5)
    # the pair (i, i+d/2) turns by pos * theta^(-2i/d), counter-clockwise
    i = 3
    ang = 7 * 10000.0 ** (-2 * i / d)
    a, b = x[0, 2, i], x[0, 2, i + d // 2]
    assert y[0, 2, i].item() == pytest.approx(a * math.cos(ang) - b * math.sin(ang), abs=1e-5)
    assert y[0, 2, i + d // 2].item() == pytest.approx(b * math.cos(ang) + a * math.sin(ang), abs=1e-5)


def test_rope_scores_depend_on_distance_only():
    d = 32
    g = torch.Generator().manual_seed(3)
    q = torch.randn(1, 1, d, generator=g)
    k = torch.randn(1, 1, d, generator=g)

    def score(m, n):
        cq, sq = P.rope_cos_sin(d, 1e6, torch.tensor([m]), torch.float64)
        ck, sk = P.rope_cos_sin(d, 1e6, torch.tensor([n]), torch.float64)
        return (P.apply_rope(q.double(), cq, sq) * P.apply_rope(k.double(), ck, sk)).sum().item()

    assert score(5, 2) == pytest.approx(score(105, 102), abs=1e-4)
    assert score(5, 2) != pytest.approx(score(5, 3), abs=1e-3)


def test_attention_is_library_sdpa_with_gqa():
    g = torch.Generator().manual_seed(4)
    nq, nkv, t, d = 6, 2, 9, 8
    q = torch.randn(nq, t, d, generator=g)
    k = torch.randn(nkv, t, d, generator=g)
    v = torch.randn(nkv, t, d, generator=g)
    ref = F.scaled_dot_product_attention(q[None], k[None], v[None], is_causal=True, enable_gqa=True)[0]
    torch.testing.assert_close(P.attention_core(q, k, v, P.causal_mask(t, t)), ref, rtol=1e-5, atol=1e-5)


def test_attention_without_mask_or_rotation_one_head_is_softmax_formula():
    g = torch.Generator().manual_seed(5)
    q = torch.randn(1, 4, 8, generator=g)
    k = torch.randn(1, 6, 8, generator=g)
    v = torch.randn(1, 6, 8, generator=g)
    ref = torch.softmax(q[0] @ k[0].T / math.sqrt(8), -1) @ v[0]
    out = P.attention_core(q, k, v, torch.ones(4, 6, dtype=torch.bool))
    torch.testing.assert_close(out[0], ref, rtol=1e-5, atol=1e-6)


def test_attention_gqa_head_map_and_single_key():
    # kv heads made distinguishable: v of kv head j is the constant j+1
    nq, nkv, t, d = 6, 2, 4, 4
    g = torch.Generator().manual_seed(6)
    q = torch.randn(nq, t, d, generator=g)
    k = torch.randn(nkv, t, d, generator=g)
    v = torch.stack([torch.full((t, d), float(j + 1)) for j in range(nkv)])
    out = P.attention_core(q, k, v, P.causal_mask(t, t))
    for h in range(nq):
        torch.testing.assert_close(out[h], torch.full((t, d), float(h // 3 + 1)))
    # first query sees one key only: output equals that key's value row
    v2 = torch.randn(nkv, t, d, generator=g)
    out2 = P.attention_core(q, k, v2, P.causal_mask(t, t))
    torch.testing.assert_close(out2[4, 0], v2[1, 0])
    # equal keys: output is the mean of the visible values
    k_eq = torch.ones(nkv, t, d)
    out3 = P.attention_core(q, k_eq, v2, P.causal_mask(t, t))
    torch.testing.assert_close(out3[0, 2], v2[0, :3].mean(0), rtol=1e-5, atol=1e-6)


def test_lens_mask_matches_reference_vector():
    """The reference's own case (tests/test_attention_backend.py:29-61): q [2,4,3,2],
    k,v [2,2,5,2], q_lens [3,1], k_lens [5,2]; the lens rule gives the explicit mask."""
    rng = np.random.default_rng(0)
    q = torch.from_numpy(rng.standard_normal((2, 4, 3, 2), dtype=np.float32))
    k = torch.from_numpy(rng.standard_normal((2, 2, 5, 2), dtype=np.float32))
    v = torch.from_numpy(rng.standard_normal((2, 2, 5, 2), dtype=np.float32))
    for b, (ql, kl) in enumerate([(3, 5), (1, 2)]):
        out = P.attention_core(q[b, :, :ql], k[b, :, :kl], v[b, :, :kl], P.causal_mask(ql, kl))
        # explicit: query i of the portion sits at absolute position kl - ql + i
        for i in range(ql):
            n_vis = kl - ql + i + 1
            full = P.attention_core(
                q[b, :, i : i + 1], k[b, :, :n_vis], v[b, :, :n_vis], torch.ones(1, n_vis, dtype=torch.bool)
            )
            torch.testing.assert_close(out[:, i : i + 1], full, rtol=1e-5, atol=1e-5)


def test_chunk_with_offset_equals_rows_of_whole():
    g = torch.Generator().manual_seed(7)
    q = torch.randn(4, 10, 8, generator=g)
    k = torch.randn(2, 10, 8, generator=g)
    v = torch.randn(2, 10, 8, generator=g)
    whole = P.attention_core(q, k, v, P.causal_mask(10, 10))
    part = P.attention_core(q[:, 6:9], k[:, :9], v[:, :9], P.causal_mask(3, 9))
    torch.testing.assert_close(part, whole[:, 6:9], rtol=1e-5, atol=1e-6)


def test_swiglu_is_library_silu():
    g = torch.Generator().manual_seed(8)
    x = torch.randn(3, 12, generator=g)
    wg, wu, wd = (torch.randn(20, 12, generator=g), torch.randn(20, 12, generator=g), torch.randn(12, 20, generator=g))
    ref = F.linear(F.silu(F.linear(x, wg)) * F.linear(x, wu), wd)
    torch.testing.assert_close(P.swiglu(wg, wu, wd, x), ref)


@pytest.mark.parametrize("tiny", [TINY_A, TINY_B], ids=["A", "B"])
def test_qk_norm_is_per_head(tiny):
    cfg = P_cfg(tiny)
    w = make_weights_dict(tiny)
    g = torch.Generator().manual_seed(9)
    t, hsz = 6, cfg["hidden_size"]
    x = torch.randn(t, hsz, generator=g)
    pos = torch.arange(t)
    p = "model.layers.0.self_attn"
    base = P.attention_block(w, p, cfg, x, pos)
    # scaling one q head's projection rows by a constant must change nothing: the per-head
    # norm divides it out (a norm over all heads at once fails; the norm's place relative to
    # the rotation is the next test's subject)
    d = cfg["head_dim"]
    w2 = dict(w)
    qw = w[f"{p}.q_proj.weight"].clone()
    qw[d : 2 * d] *= 5.0
    w2[f"{p}.q_proj.weight"] = qw
    # (up to eps, which does not scale with the head: hence the absolute slack)
    torch.testing.assert_close(P.attention_block(w2, p, cfg, x, pos), base, rtol=1e-4, atol=2e-5)
    # while scaling one *element* inside a head does change it
    qw3 = w[f"{p}.q_proj.weight"].clone()
    qw3[d] *= 5.0
    w3 = dict(w)
    w3[f"{p}.q_proj.weight"] = qw3
    assert not torch.allclose(P.attention_block(w3, p, cfg, x, pos), base, rtol=1e-3, atol=1e-4)


def P_cfg(tiny):
    c = dict(tiny["config"])
    nq = c["num_attention_heads"]
    return dict(
        vocab_size=c["vocab_size"], hidden_size=c["hidden_size"], intermediate_size=c["intermediate_size"],
        num_hidden_layers=c["num_hidden_layers"], num_heads=nq, num_kv_heads=c["num_key_value_heads"],
        head_dim=c["head_dim"], rms_norm_eps=c["rms_norm_eps"], rope_theta=c["rope_theta"],
        tie_word_embeddings=c["tie_word_embeddings"],
    )


@pytest.mark.parametrize("tiny", [TINY_A, TINY_B], ids=["A", "B"])
def test_forward_shift_invariance_and_causality(tiny):
    cfg = P_cfg(tiny)
    w = make_weights_dict(tiny)
    rng = np.random.default_rng(3)
    ids = rng.integers(0, cfg["vocab_size"], size=21).tolist()
    base = P.forward(w, cfg, ids)
    assert base.shape == (21, cfg["vocab_size"])
    # only distances count: shifting every position leaves the logits alone
    shifted = P.forward(w, cfg, ids, first_position=37)
    torch.testing.assert_close(shifted, base, rtol=2e-3, atol=2e-4)
    # causal: a later token does not change earlier logits
    ids2 = list(ids)
    ids2[-1] = (ids2[-1] + 1) % cfg["vocab_size"]
    torch.testing.assert_close(P.forward(w, cfg, ids2)[:-1], base[:-1])
    # prefix property: forward of a prefix gives the same rows
    torch.testing.assert_close(P.forward(w, cfg, ids[:9]), base[:9], rtol=1e-4, atol=1e-5)


def test_tied_head_uses_embedding_table():
    cfg = P_cfg(TINY_A)
    assert cfg["tie_word_embeddings"]
    w = make_weights_dict(TINY_A)
    ids = [1, 2, 3]
    base = P.forward(w, cfg, ids)
    w2 = dict(w)
    w2["lm_head.weight"] = torch.zeros_like(w["model.embed_tokens.weight"])  # must be ignored when tied
    torch.testing.assert_close(P.forward(w2, cfg, ids), base)


def test_greedy_generate_stops_on_eos_and_counts_it():
    cfg = P_cfg(TINY_A)
    w = make_weights_dict(TINY_A)
    out = P.greedy_generate(w, cfg, [5, 6, 7], 6)
    assert len(out) == 6
    out2 = P.greedy_generate(w, cfg, [5, 6, 7], 6, eos_id=out[2])
    first = out.index(out[2])
    assert out2 == out[: first + 1]


def test_forward_scheduled_reduces_to_forward_and_window_is_a_band():
    cfg = P_cfg(TINY_B)
    w = make_weights_dict(TINY_B)
    ids = list(range(3, 30))
    base = P.forward(w, cfg, ids)
    plain_order = [(i, None) for i in range(cfg["num_hidden_layers"])]
    torch.testing.assert_close(P.forward_scheduled(w, cfg, ids, plain_order), base)
    # a window at least as long as the sequence changes nothing; a short one changes late rows only
    torch.testing.assert_close(P.forward_scheduled(w, cfg, ids, plain_order, {0: 27, 1: 100}), base)
    short = P.forward_scheduled(w, cfg, ids, plain_order, {1: 5})
    torch.testing.assert_close(short[:5], base[:5])
    assert not torch.allclose(short[10:], base[10:], rtol=1e-3, atol=1e-4)


# ---- how the parts are put together.  The reference has no tiny model with q/k norms or with
# norm weights other than one (its tests/_tiny_model.py:20-97 is Qwen2-typed), and model code of
# other packages is no source here, so the composition is pinned by invariants that a plausible
# other arrangement breaks; every test below shows that its mutant really fails.
def _strong_qk_weights(tiny, seed):
    """Weights whose q/k norm weights differ strongly inside every rotated pair (i, i + D/2)."""
    w = make_weights_dict(tiny)
    d = tiny["config"]["head_dim"]
    g = torch.Generator().manual_seed(seed)
    for name in list(w):
        if name.endswith("q_norm.weight") or name.endswith("k_norm.weight"):
            w[name] = torch.cat([2.0 + torch.rand(d // 2, generator=g), 0.2 + 0.2 * torch.rand(d // 2, generator=g)])
    return w


def _attention_with_norm_after_rotation(w, p, cfg, x, positions):
    """The mutant: the same block with the per-head norm applied after the rotation."""
    t = x.shape[0]
    nq, nkv, d = cfg["num_heads"], cfg["num_kv_heads"], cfg["head_dim"]
    cos, sin = P.rope_cos_sin(d, cfg["rope_theta"], positions, x.dtype)
    q = P.linear(w[f"{p}.q_proj.weight"], x).reshape(t, nq, d).transpose(0, 1)
    k = P.linear(w[f"{p}.k_proj.weight"], x).reshape(t, nkv, d).transpose(0, 1)
    v = P.linear(w[f"{p}.v_proj.weight"], x).reshape(t, nkv, d).transpose(0, 1)
    q = P.rms_norm(w[f"{p}.q_norm.weight"], cfg["rms_norm_eps"], P.apply_rope(q, cos, sin))
    k = P.rms_norm(w[f"{p}.k_norm.weight"], cfg["rms_norm_eps"], P.apply_rope(k, cos, sin))
    out = P.attention_core(q, k, v, P.causal_mask(t, t)).transpose(0, 1).reshape(t, nq * d)
    return P.linear(w[f"{p}.o_proj.weight"], out)


@pytest.mark.parametrize("tiny", [TINY_A, TINY_B], ids=["A", "B"])
def test_qk_norm_comes_before_the_rotation(tiny):
    """jllm/model/common.py:107-111 then :130-131: norm, then rotation.  Only then is the rotated
    vector a rotation of something that does not depend on the position, so that scores depend on
    distances alone and a shift of all positions changes nothing.  A norm weight applied after
    the rotation scales the two elements of a pair differently, which is no rotation any more:
    the mutant's output moves with the shift."""
    cfg = P_cfg(tiny)
    w = _strong_qk_weights(tiny, 11)
    g = torch.Generator().manual_seed(12)
    x = torch.randn(9, cfg["hidden_size"], generator=g)
    p = "model.layers.0.self_attn"
    here, there = torch.arange(9), torch.arange(9) + 23
    base = P.attention_block(w, p, cfg, x, here)
    torch.testing.assert_close(P.attention_block(w, p, cfg, x, there), base, rtol=1e-4, atol=1e-5 * float(base.abs().max()) + 1e-6)
    mutant_here = _attention_with_norm_after_rotation(w, p, cfg, x, here)
    mutant_there = _attention_with_norm_after_rotation(w, p, cfg, x, there)
    scale = float(base.abs().max())
    assert float((mutant_there - mutant_here).abs().max()) > 0.02 * scale      # the mutant is not shift invariant
    assert float((mutant_here - base).abs().max()) > 0.02 * scale              # and is another function altogether


def test_qk_norm_takes_the_models_eps():
    """jllm/model/weights.py:128-129: the q/k norms are built with the model's rms_norm_eps.
    With an input so small that the mean square of a head is of eps's order, the output depends
    on eps: a constant written into the block instead of the configuration's value would not."""
    cfg = P_cfg(TINY_B)
    w = make_weights_dict(TINY_B)
    g = torch.Generator().manual_seed(13)
    x = 0.05 * torch.randn(7, cfg["hidden_size"], generator=g)
    p = "model.layers.1.self_attn"
    q = P.linear(w[f"{p}.q_proj.weight"], x)
    ms = float((q * q).mean())
    outs = [P.attention_block(w, p, dict(cfg, rms_norm_eps=e), x, torch.arange(7)) for e in (0.0, ms, 100 * ms)]
    assert not torch.allclose(outs[0], outs[1], rtol=1e-2, atol=0) and not torch.allclose(outs[1], outs[2], rtol=1e-2, atol=0)
    # eps -> infinity silences q and k: every visible key then weighs the same (scores -> 0)
    t = 7
    v = P.linear(w[f"{p}.v_proj.weight"], x).reshape(t, cfg["num_kv_heads"], cfg["head_dim"]).transpose(0, 1)
    flat = P.attention_block(w, p, dict(cfg, rms_norm_eps=1e12), x, torch.arange(t))
    mean_v = torch.cumsum(v, dim=1) / torch.arange(1, t + 1)[None, :, None]
    rep = cfg["num_heads"] // cfg["num_kv_heads"]
    want = torch.repeat_interleave(mean_v, rep, dim=0).transpose(0, 1).reshape(t, -1) @ w[f"{p}.o_proj.weight"].T
    torch.testing.assert_close(flat, want, rtol=1e-3, atol=1e-6)


@pytest.mark.parametrize("tiny", [TINY_A, TINY_B], ids=["A", "B"])
def test_layer_is_prenorm_residual_and_sequential(tiny):
    """jllm/model/common.py:140-147: h += mixer(norm_1(h)); h += feed_forward(norm_2(h)).
    Invariants: (1) the residual passes through unnormed and each sublayer sees a normed input:
    with the feed-forward silenced, layer(c*h) - c*h does not depend on c (a post-norm layer,
    norm(h + f(h)), fails this); (2) the feed-forward reads the stream *after* the mixer's output
    was added: doubling the mixer's output changes more than the mixer's share (a parallel layer,
    h + f(norm h) + g(norm h), fails this); (3) with both sublayers silenced the layer is the
    identity."""
    cfg = P_cfg(tiny)
    w = make_weights_dict(tiny)
    g = torch.Generator().manual_seed(14)
    t = 6
    h = torch.randn(t, cfg["hidden_size"], generator=g)
    pos = torch.arange(t)
    p = "model.layers.0"
    quiet_ffn = dict(w, **{f"{p}.mlp.down_proj.weight": torch.zeros_like(w[f"{p}.mlp.down_proj.weight"])})
    quiet_mixer = dict(w, **{f"{p}.self_attn.o_proj.weight": torch.zeros_like(w[f"{p}.self_attn.o_proj.weight"])})
    quiet_both = dict(quiet_ffn, **{f"{p}.self_attn.o_proj.weight": quiet_mixer[f"{p}.self_attn.o_proj.weight"]})
    torch.testing.assert_close(P.decoder_layer(quiet_both, 0, cfg, h, pos), h)
    # (1) mixer share is the same for h and 40*h (up to eps)
    a1 = P.decoder_layer(quiet_ffn, 0, cfg, h, pos) - h
    a40 = P.decoder_layer(quiet_ffn, 0, cfg, 40 * h, pos) - 40 * h
    assert float(a1.abs().max()) > 1e-3
    torch.testing.assert_close(a40, a1, rtol=2e-3, atol=2e-3 * float(a1.abs().max()))
    f1 = P.decoder_layer(quiet_mixer, 0, cfg, h, pos) - h
    f40 = P.decoder_layer(quiet_mixer, 0, cfg, 40 * h, pos) - 40 * h
    torch.testing.assert_close(f40, f1, rtol=2e-3, atol=2e-3 * float(f1.abs().max()))
    # the shares use their own norm weights: input_layernorm feeds the mixer, post_attention_layernorm the feed-forward
    for name, quiet, moves in ((f"{p}.input_layernorm.weight", quiet_ffn, True), (f"{p}.post_attention_layernorm.weight", quiet_ffn, False),
                               (f"{p}.input_layernorm.weight", quiet_mixer, False), (f"{p}.post_attention_layernorm.weight", quiet_mixer, True)):
        changed = dict(quiet, **{name: quiet[name].flip(0) * 1.5})
        same = torch.allclose(P.decoder_layer(changed, 0, cfg, h, pos), P.decoder_layer(quiet, 0, cfg, h, pos), rtol=1e-4, atol=1e-6)
        assert same != moves, (name, moves)
    # (2) sequential: make the mixer's output as large as the stream, then double it
    big = dict(w, **{f"{p}.self_attn.o_proj.weight": w[f"{p}.self_attn.o_proj.weight"] * (float(h.abs().mean()) / float(a1.abs().mean()))})
    big2 = dict(big, **{f"{p}.self_attn.o_proj.weight": big[f"{p}.self_attn.o_proj.weight"] * 2})
    a = P.decoder_layer(dict(big, **{f"{p}.mlp.down_proj.weight": quiet_ffn[f"{p}.mlp.down_proj.weight"]}), 0, cfg, h, pos) - h
    diff = P.decoder_layer(big2, 0, cfg, h, pos) - P.decoder_layer(big, 0, cfg, h, pos)
    ffn_scale = float((P.decoder_layer(big, 0, cfg, h, pos) - h - a).abs().max())
    assert float((diff - a).abs().max()) > 0.05 * ffn_scale      # the feed-forward's input moved with the mixer's output


@pytest.mark.parametrize("tiny", [TINY_A, TINY_B], ids=["A", "B"])
def test_final_norm_sits_between_the_last_layer_and_the_head(tiny):
    """jllm/model/common.py:168-170: logits = head(norm(h)).  With every sublayer silenced the
    model is head(norm(embed)): the logits then do not depend on the scale of the embedding rows
    (no final norm, or a norm after the head, fails), are linear in the final norm's weight, and
    equal the library's rms_norm and linear applied to the embedding rows."""
    cfg = P_cfg(tiny)
    w = make_weights_dict(tiny)
    for name in list(w):
        if name.endswith("o_proj.weight") or name.endswith("down_proj.weight"):
            w[name] = torch.zeros_like(w[name])
    if cfg["tie_word_embeddings"]:
        pytest.skip("a tied head moves with the embedding rows")
    ids = [3, 1, 4, 1, 5, 9, 2, 6]
    base = P.forward(w, cfg, ids)
    # (rows made large first, so that eps is nothing beside their mean square)
    large = dict(w, **{"model.embed_tokens.weight": 30 * w["model.embed_tokens.weight"]})
    larger = dict(w, **{"model.embed_tokens.weight": 900 * w["model.embed_tokens.weight"]})
    torch.testing.assert_close(P.forward(larger, cfg, ids), P.forward(large, cfg, ids), rtol=1e-4,
                               atol=1e-4 * float(base.abs().max()))
    assert float((P.forward(large, cfg, ids) - base).abs().max()) < 0.01 * float(base.abs().max())
    doubled = dict(w, **{"model.norm.weight": 2 * w["model.norm.weight"]})
    torch.testing.assert_close(P.forward(doubled, cfg, ids), 2 * base)
    e = w["model.embed_tokens.weight"][torch.tensor(ids)]
    want = F.linear(F.rms_norm(e, (cfg["hidden_size"],), w["model.norm.weight"], cfg["rms_norm_eps"]), w["lm_head.weight"])
    torch.testing.assert_close(base, want, rtol=1e-5, atol=1e-6)


def test_last_logits_row_and_greedy_rollout_agree_with_prefix_recomputation():
    """What the reference's parity tests hold against another implementation, held here against
    the oracle's own prefix property (tests/test_long_rollout.py:19-36: 40 tokens, exact): the
    token at step i is the argmax of the last row of forward(prompt + tokens[:i]), whether that
    row is computed with the whole sequence or read off a longer one."""
    cfg = P_cfg(TINY_B)
    w = make_weights_dict(TINY_B)
    prompt = [7, 300, 12, 45, 2]
    out = P.greedy_generate(w, cfg, prompt, 40)
    full = P.forward(w, cfg, prompt + out)
    assert [int(full[len(prompt) - 1 + i].argmax()) for i in range(40)] == out


@pytest.mark.parametrize("tiny", [TINY_B, TINY_C], ids=["B", "C"])
def test_attention_block_splits_heads_row_block_by_row_block_and_joins_them_head_major(tiny):
    """With ``o_proj`` set to select the D columns of query head j, the block's output is the
    library's attention of that head alone: q from rows [jD, (j+1)D) of ``q_proj``, k and v from
    rows [gD, (g+1)D) of ``k_proj`` / ``v_proj`` with g = j // (heads per kv head), each after the
    library's ``rms_norm`` over D and the rotation pinned above.  A head split taken from the wrong
    axis (interleaved heads), a kv head map j % nkv, or a concat that is not head-major fails it."""
    c = tiny["config"]
    nq, nkv, d, hid = c["num_attention_heads"], c["num_key_value_heads"], c["head_dim"], c["hidden_size"]
    cfg = dict(num_heads=nq, num_kv_heads=nkv, head_dim=d, rms_norm_eps=c["rms_norm_eps"], rope_theta=c["rope_theta"])
    w = {k.replace("model.layers.0.self_attn", "p"): v.double() for k, v in make_weights_dict(tiny).items()
         if k.startswith("model.layers.0.self_attn")}
    t = 11
    g = torch.Generator().manual_seed(44)
    x = torch.randn(t, hid, generator=g, dtype=torch.float64)
    pos = torch.arange(t) + 3
    cos, sin = P.rope_cos_sin(d, c["rope_theta"], pos, torch.float64)
    for j in range(nq):
        kv = j // (nq // nkv)
        select = torch.zeros(d, nq * d, dtype=torch.float64)
        select[torch.arange(d), j * d + torch.arange(d)] = 1.0
        out = P.attention_block(dict(w, **{"p.o_proj.weight": select}), "p", cfg, x, pos)
        q = F.rms_norm(x @ w["p.q_proj.weight"][j * d:(j + 1) * d].T, (d,), w["p.q_norm.weight"], c["rms_norm_eps"])
        k = F.rms_norm(x @ w["p.k_proj.weight"][kv * d:(kv + 1) * d].T, (d,), w["p.k_norm.weight"], c["rms_norm_eps"])
        v = x @ w["p.v_proj.weight"][kv * d:(kv + 1) * d].T
        q, k = P.apply_rope(q[None], cos, sin), P.apply_rope(k[None], cos, sin)
        ref = F.scaled_dot_product_attention(q[None], k[None], v[None, None], is_causal=True)[0, 0]
        torch.testing.assert_close(out, ref, rtol=1e-9, atol=1e-9)
