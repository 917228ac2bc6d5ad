"""The layer sizes of real models (Qwen3-8B: hidden 4096, 32/8 heads of 128, feed-forward
12288, vocabulary 151936; the 14B sizes: hidden 5120, 40/8 heads, feed-forward 17408; the 32B
sizes: hidden 5120, 64/8 heads, so that heads * head size = 8192 is not the width, feed-forward
25600) with two layers of random weights: the 32-bit path and the bfloat16
path against the plain implementation, whole, token by token, in portions and mixed.  These are
the sizes at which the kernels' wide paths run (16-byte norm loads, the streaming matrix
product's real shapes, a vocabulary that is no power of two, the 128-wide MFMA attention).

Then the shapes that the measurement program times, again against the plain implementation:
decode-only steps of 8, 24 and 64 requests behind prompts of about 1,024 tokens, recorded and
replayed and started ahead of their tokens; one prompt of 2,048 tokens whole, cut, and behind a
prefix taken from the cache; contexts of 8,300 and 20,000 tokens on a narrow model with the real
head geometry; one far token that decides the logits; and the workloads of the larger
configurations: running decodes joined by long prompts in portions with a shared prefix (14B
sizes), decodes behind 16,400 tokens (32B sizes).  The plain implementation runs on the GPU here,
in torch's exact float32."""
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
# the real head geometry (4 query heads of 128 per kv head, page 16) on a narrow model: long contexts stay cheap
CONFIG_NARROW = dict(CONFIG, hidden_size=512, num_attention_heads=8, num_key_value_heads=2, intermediate_size=1536,
                     vocab_size=3000)


class Sized:
    """Random weights of one configuration on the GPU (rounded through bfloat16 like a stored
    checkpoint): bound models of either type, and the plain implementation's float copy."""

    def __init__(self, config, seed=0):
        from jax_vllm_amd.config import resolve
        from jax_vllm_amd.parts import DecoderModel
        from jax_vllm_amd.weights.random_init import _draw

        P.use_exact_float32_products()
        arch, cfg, _ = resolve(config)
        self.cfg, self.spec = cfg, arch.build_spec(cfg)
        self.names = DecoderModel(self.spec).tensor_specs()
        self.dev = {n: _draw(ts, seed, n, 0.02, 0.02, device="cuda").to(torch.bfloat16) for n, ts in self.names.items()}
        self.plain_w = {n: t.float() for n, t in self.dev.items()}
        self.plain_cfg = dict(
            vocab_size=cfg.vocab_size, hidden_size=cfg.hidden_size, intermediate_size=cfg.intermediate_size,
            num_hidden_layers=cfg.num_hidden_layers, num_heads=cfg.num_heads, num_kv_heads=cfg.num_kv_heads,
            head_dim=cfg.head_dim, rms_norm_eps=cfg.rms_norm_eps, rope_theta=cfg.rope_theta,
            tie_word_embeddings=cfg.tie_word_embeddings)
        self._models = {}

    def model(self, dtype):
        from jax_vllm_amd.parts import DecoderModel
        from jax_vllm_amd.weights.loader import target_dtype

        if dtype not in self._models:
            compute = torch.float32 if dtype == "float32" else torch.bfloat16
            m = DecoderModel(self.spec)
            m.bind({n: self.dev[n].to(target_dtype(self.names[n].role, compute)).contiguous() for n in self.names}, compute)
            self._models[dtype] = m
        return self._models[dtype]

    def plain(self, tokens, rows=None) -> np.ndarray:
        return P.forward(self.plain_w, self.plain_cfg, tokens, rows=rows).cpu().numpy()


@pytest.fixture(scope="module", params=[CONFIG, CONFIG_14B, CONFIG_32B], ids=["8b", "14b", "32b"])
def big(request):
    sized = Sized(request.param)
    rng = np.random.default_rng(0)
    reqs = {f"r{i}": rng.integers(0, sized.cfg.vocab_size, size=n).tolist() for i, n in enumerate((64, 150, 300, 97))}
    want = {r: sized.plain(t) for r, t in reqs.items()}
    if request.param is CONFIG:
        # the oracle on the GPU is the oracle on the CPU: same formulas, exact float32 products
        on_cpu = P.forward({n: t.cpu() for n, t in sized.plain_w.items()}, sized.plain_cfg, reqs["r0"]).numpy()
        scale = float(np.abs(on_cpu).max())
        assert float(np.abs(on_cpu - want["r0"]).max()) <= 1e-5 * scale
    yield sized.model, reqs, want
    del sized
    torch.cuda.empty_cache()


def every_cut(core, reqs, want, dtype, check_logits=check_logits) -> float:
    """Each request whole; one with its last 32 tokens one by one; all four in portions of changing
    size beside single tokens of the others.  Returns the largest error seen, as a fraction of the
    largest logit."""
    from jax_vllm_amd.engine.entries import StepEntry

    scale = max(float(np.abs(w).max()) for w in want.values())
    errs = []

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
        errs.append(check_logits(dtype, run([(r, toks)])[0], want[r], scale, f"{r} whole"))
        core.finish_request(r)
    r, toks = "r1", reqs["r1"]
    core.start_request(r)
    got = run([(r, toks[:-32])])
    for i in range(len(toks) - 32, len(toks)):
        got += run([(r, toks[i:i + 1])])
    errs.append(check_logits(dtype, np.concatenate(got), want[r], scale, f"{r} tail one by one"))
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
        errs.append(check_logits(dtype, np.concatenate(got[r]), want[r], scale, f"{r} mixed"))
        core.finish_request(r)
    core.cache.check_invariants()
    return max(errs) / scale


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_real_layer_sizes_every_cut(big, dtype):
    model, reqs, want = big
    # replayed steps here are those of one row (the tail one by one); more rows: the tests of the benchmark's shapes below
    core = make_core(None, dtype, 16, pages=48, seqs=4, model=model(dtype), graphs=(dtype == "bfloat16"))
    every_cut(core, reqs, want, dtype)


def test_all_36_layers_of_the_8b_sizes_every_cut(capsys):
    """The whole depth of the configuration that the measurement program runs, once: 36 layers of
    the 8B sizes, 4 prompts of 64 to 300 tokens, whole / last 32 tokens one by one / portions /
    mixed.  Rounding errors add up like a random walk over the layers (measured against the plain
    implementation in float64, as a fraction of the largest logit: the plain float32 implementation
    itself 0.5e-5 at 2 layers, 1.4e-5 at 12, 2.2e-5 at 36; the 32-bit engine 0.6e-5, 1.3e-5, 2.3e-5;
    the bfloat16 engine 1.2e-2, 2.6e-2, 4.4e-2 with cosines from 0.9999 down to 0.9988), so at this
    depth the oracle is the float64 one and the bounds are: 32-bit engine 4e-5 and at most twice the
    plain float32 implementation's own error; bfloat16 engine 6e-2 and cosine 0.998 (the bar of the
    reference's own bfloat16 test, tests/test_parity.py:26-29 there)."""
    sized = Sized(dict(CONFIG, num_hidden_layers=36))
    rng = np.random.default_rng(0)
    reqs = {f"r{i}": rng.integers(0, sized.cfg.vocab_size, size=n).tolist() for i, n in enumerate((64, 150, 300, 97))}
    w64 = {n: t.double() for n, t in sized.plain_w.items()}
    want = {r: P.forward(w64, sized.plain_cfg, t).cpu().numpy() for r, t in reqs.items()}
    del w64
    scale = max(float(np.abs(w).max()) for w in want.values())
    plain32 = max(float(np.abs(sized.plain(t) - want[r]).max()) for r, t in reqs.items())
    assert plain32 <= 3e-5 * scale

    def deep_check(dtype, got, want, scale=None, what=""):
        err = float(np.abs(np.asarray(got, dtype=np.float64) - want).max())
        if dtype == "float32":
            assert err <= 4e-5 * scale and err <= 2 * plain32, f"{what}: max error {err} (scale {scale}, plain float32 {plain32})"
        else:
            assert err <= 6e-2 * scale, f"{what}: max error {err} (scale {scale})"
            g, w = np.asarray(got, dtype=np.float64), want
            cos = (g * w).sum(-1) / (np.linalg.norm(g, axis=-1) * np.linalg.norm(w, axis=-1) + 1e-30)
            assert cos.min() >= 0.998, f"{what}: cosine {cos.min()}"
        return err

    for dtype in ("float32", "bfloat16"):
        core = make_core(None, dtype, 16, pages=48, seqs=4, model=sized.model(dtype), graphs=True)
        err = every_cut(core, reqs, want, dtype, check_logits=deep_check)
        with capsys.disabled():
            print(f"\n[36 layers, {dtype}] largest error / largest logit = {err:.3e} (plain float32: {plain32 / scale:.3e})",
                  flush=True)
        del core
        sized._models.clear()
        torch.cuda.empty_cache()


# ------------------------------------------------------------------ the shapes that the measurement program times
@pytest.fixture(scope="module")
def sized_8b():
    sized = Sized(CONFIG)
    yield sized
    del sized
    torch.cuda.empty_cache()


DECODE_STEPS = 12


@pytest.mark.parametrize("dtype,batch", [("bfloat16", 8), ("bfloat16", 24), ("bfloat16", 64), ("float32", 8), ("float32", 24), ("float32", 64)])
def test_decode_steps_of_many_requests_behind_long_prompts_replayed_and_started_ahead(sized_8b, dtype, batch):
    """What the decode benchmark times: ``batch`` requests behind prompts of 1,000 to 1,060 tokens
    (prefilled under a budget of 2,048 tokens a step), then decode-only steps of all of them,
    recorded, replayed and started ahead of their tokens.  First through the entry point: every
    token must be the plain implementation's choice.  Then the same kind of steps through the step
    function with given tokens: every row's logits against the plain ones."""
    from jax_vllm_amd.engine.entries import StepEntry
    from jax_vllm_amd.engine.llm import LLM
    from jax_vllm_amd.engine.request import SamplingParams

    sized = sized_8b
    vocab = sized.cfg.vocab_size
    rng = np.random.default_rng(100 + batch)
    lens = rng.integers(1000, 1061, size=batch).tolist()
    prompts = [rng.integers(0, vocab, size=n).tolist() for n in lens]
    llm = LLM(sized.model(dtype), dtype=dtype, max_num_seqs=batch, max_model_len=1280, max_num_batched_tokens=2048,
              block_size=16, use_hip_graphs=True, decode_ahead=True, enable_prefix_cache=False)
    rids = [llm.add_request(p, SamplingParams(max_new_tokens=200)) for p in prompts]
    outs = {r: [] for r in rids}

    def step():
        events = llm.step()
        for e in events:
            outs[e.request_id].append(e.token)
        return len(events)

    # as the measurement does: prompts two a step beside the decodes of those that are through, untimed there ...
    while llm.scheduler.waiting or any(r.num_remaining > 1 or not r.output_ids for r in llm.scheduler.running):
        step()
    before = (llm.stats.graph_replays, llm.stats.steps_ahead)
    for _ in range(DECODE_STEPS):            # ... then the steps it times: one token of every request
        assert step() == batch
    assert llm.stats.graph_replays - before[0] >= DECODE_STEPS - 2 and llm.stats.steps_ahead - before[1] >= DECODE_STEPS - 2
    assert llm.stats.preemptions == 0
    llm.abort_all()
    tight = dtype == "float32"
    for i, (p, rid) in enumerate(zip(prompts, rids)):
        out = outs[rid]
        assert len(out) >= DECODE_STEPS + 1
        rows = list(range(len(p) - 1, len(p) + len(out) - 1))
        logits = sized.plain(p + out[:-1], rows)
        for k, t in enumerate(out):
            margin = float(logits[k].max() - logits[k][t])
            allowed = (1e-4 if tight else 0.04) * float(np.abs(logits[k]).max())
            assert margin <= allowed, f"request {i}, token {k}: engine's {t} is {margin} below the plain maximum"

    # the step function itself, with given tokens, so that every row's logits can be compared
    core = llm.core
    assert not core.cache.requests
    replays_before = core.graph_replays
    tails = [rng.integers(0, vocab, size=DECODE_STEPS).tolist() for _ in range(batch)]
    ids = [f"q{i}" for i in range(batch)]
    got = {r: [] for r in ids}
    for r in ids:
        core.start_request(r)
    for first in range(0, batch, 2):         # two prompts a step: about 2,048 tokens
        pair = list(range(first, min(first + 2, batch)))
        out = core.run([StepEntry(ids[i], prompts[i], [len(prompts[i]) - 1]) for i in pair]).cpu().numpy()
        for k, i in enumerate(pair):
            got[ids[i]].append(out[k:k + 1])
    for step in range(DECODE_STEPS):
        out = core.run([StepEntry(ids[i], [tails[i][step]], [0]) for i in range(batch)]).cpu().numpy()
        for i in range(batch):
            got[ids[i]].append(out[i:i + 1])
    assert core.graph_replays - replays_before >= DECODE_STEPS - 1
    scale = None
    for i in range(batch):
        rows = list(range(lens[i] - 1, lens[i] + DECODE_STEPS))
        want = sized.plain(prompts[i] + tails[i], rows)
        scale = scale or float(np.abs(want).max())
        check_logits(dtype, np.concatenate(got[ids[i]]), want, scale, f"request {i} of {batch}")
        core.finish_request(ids[i])
    core.cache.check_invariants()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_prompt_of_2048_tokens_whole_cut_and_behind_a_cached_prefix(sized_8b, dtype):
    """What the prefill benchmark times: one prompt of 2,048 tokens in one step; the same prompt as
    1,500 + 548; and a second prompt that shares its first 1,504 tokens, which are then found in
    the cache, so that only 544 tokens run, behind pages that another request wrote.  Logits at 64
    places spread over the prompt (page and tile edges among them)."""
    from jax_vllm_amd.engine.entries import StepEntry

    sized = sized_8b
    rng = np.random.default_rng(7)
    n = 2048
    prompt = rng.integers(0, sized.cfg.vocab_size, size=n).tolist()
    rows = sorted(set(np.linspace(0, n - 1, 50).astype(int).tolist()
                      + [1, 15, 16, 63, 64, 127, 128, 1023, 1024, 1499, 1500, 1501, 1503, 1504, 1505, 2046]))[:64]
    assert len(rows) == 64
    want = sized.plain(prompt, rows)
    scale = float(np.abs(want).max())
    core = make_core(None, dtype, 16, pages=400, seqs=3, model=sized.model(dtype), prefix=True)
    core.start_request("whole", prompt)
    check_logits(dtype, core.run([StepEntry("whole", prompt, rows)]).cpu().numpy(), want, scale, "whole")
    # the pages of "whole" are hashed now; a request that is started without its prompt does not look for them
    core.start_request("cut")
    first = [r for r in rows if r < 1500]
    got = [core.run([StepEntry("cut", prompt[:1500], first)]).cpu().numpy(),
           core.run([StepEntry("cut", prompt[1500:], [r - 1500 for r in rows if r >= 1500])]).cpu().numpy()]
    check_logits(dtype, np.concatenate(got), want, scale, "1,500 + 548")
    other = prompt[:1504] + rng.integers(0, sized.cfg.vocab_size, size=n - 1504).tolist()
    assert core.start_request("behind", other) == 1504
    late = [r for r in rows if r >= 1504]
    got = core.run([StepEntry("behind", other[1504:], [r - 1504 for r in late])]).cpu().numpy()
    check_logits(dtype, got, sized.plain(other, late), scale, "544 behind 1,504 cached")
    for r in ("whole", "cut", "behind"):
        core.finish_request(r)
    core.cache.check_invariants()


@pytest.mark.parametrize("dtype,length", [("float32", 8300), ("bfloat16", 8300), ("bfloat16", 20000)])
def test_long_contexts_with_the_real_head_geometry(dtype, length):
    """One request of 8,300 (20,000) tokens in portions of 2,048, then 32 tokens one by one (replayed
    steps), on a narrow model with heads of 128, 4 per kv head, pages of 16: every position's logits."""
    from jax_vllm_amd.engine.entries import StepEntry

    sized = Sized(CONFIG_NARROW, seed=5)
    rng = np.random.default_rng(length)
    toks = rng.integers(0, sized.cfg.vocab_size, size=length + 32).tolist()
    want = sized.plain(toks)
    core = make_core(None, dtype, 16, pages=-(-(length + 32) // 16) + 2, seqs=2, model=sized.model(dtype), graphs=True)
    core.start_request("a")
    got = []
    for at in range(0, length, 2048):
        part = toks[at:min(at + 2048, length)]
        got.append(core.run([StepEntry("a", part, range(len(part)))]).cpu().numpy())
    for i in range(length, length + 32):
        got.append(core.run([StepEntry("a", toks[i:i + 1], [0])]).cpu().numpy())
    assert core.graph_replays >= 30
    check_logits(dtype, np.concatenate(got), want, what=f"{length} tokens")
    core.finish_request("a")
    core.cache.check_invariants()


# ------------------------------------------------------------------ one far token decides the logits
NEEDLE_CONFIG = dict(CONFIG, num_hidden_layers=1, hidden_size=256, num_attention_heads=4, num_key_value_heads=2,
                     intermediate_size=384, vocab_size=96)


def needle_model():
    """A one-layer model with heads of 128 whose weights are made so that ONE far token decides the last token's
    logits: token NEEDLE's key and token ASK's query are both concentrated on the head element that the rotation
    turns slowest, their q/k-norm weight there is 1.5, so ASK's score with NEEDLE is 11.3 * 1.5^2 = 25 while its
    scores with the thousands of other keys stay below 8: ASK's attention output is NEEDLE's value, whatever else
    the context holds.  Among random weights alone a lost page would move nothing that a bfloat16 bound sees."""
    sized = Sized(NEEDLE_CONFIG, seed=9)
    d, hid = 128, 256
    slow = d // 2 - 1                                        # pairs with element d - 1; angle 1e6^(-126/128) a position
    g = torch.Generator().manual_seed(3)
    w = {n: t.clone() for n, t in sized.plain_w.items()}
    p = "model.layers.0."
    needle, ask = 90, 91
    emb = 0.3 * torch.randn(96, hid, generator=g)
    emb[:, :2] = 0.0
    emb[needle] = 0.05 * torch.randn(hid, generator=g)
    emb[needle, 0] = 4.0
    emb[ask] = 0.05 * torch.randn(hid, generator=g)
    emb[ask, 1] = 4.0
    w["model.embed_tokens.weight"] = emb.cuda()
    w[p + "input_layernorm.weight"] = torch.ones(hid).cuda()
    for name, col, heads in (("k_proj", 0, 2), ("q_proj", 1, 4)):
        m = 0.05 * torch.randn(heads * d, hid, generator=g)
        m[:, :2] = 0.0
        for h in range(heads):
            m[h * d + slow, col] = 1.0
        w[p + f"self_attn.{name}.weight"] = m.cuda()
    for name in ("q_norm", "k_norm"):
        v = torch.ones(d)
        v[slow] = 1.5
        w[p + f"self_attn.{name}.weight"] = v.cuda()
    w[p + "self_attn.v_proj.weight"] = (0.3 * torch.randn(2 * d, hid, generator=g)).cuda()
    w[p + "self_attn.o_proj.weight"] = (0.3 * torch.randn(hid, 4 * d, generator=g)).cuda()
    w["lm_head.weight"] = (0.3 * torch.randn(96, hid, generator=g)).cuda()
    sized.dev = {n: t.to(torch.bfloat16) for n, t in w.items()}
    sized.plain_w = {n: t.float() for n, t in sized.dev.items()}
    return sized, needle, ask


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("context,place", [(3000, 0), (3000, 1535), (3000, 1536), (3000, 2990), (700, 351), (5000, 4097)])
def test_one_far_token_decides_the_logits(dtype, context, place):
    """The prompt holds NEEDLE once, at ``place``; ASK comes as the last token of the last prompt portion, then as a
    decoded token (a replayed step whose keys are shared out to several blocks), then once more after two other
    tokens.  The oracle says that each of these rows depends on the needle (without it the logits move by more than a
    quarter of their size), so an engine that loses, misplaces or misweights that one key among thousands is far
    outside the bound of either precision."""
    from jax_vllm_amd.engine.entries import StepEntry

    sized, needle, ask = needle_model()
    rng = np.random.default_rng(context + place)
    toks = rng.integers(0, 90, size=context).tolist()
    toks[place] = needle
    toks += [ask, ask, 5, 17, ask]
    rows = [context, context + 1, context + 4]
    want = sized.plain(toks, rows)
    without = list(toks)
    without[place] = 7
    moved = np.abs(sized.plain(without, rows) - want).max(axis=1)
    scale = float(np.abs(want).max())
    assert (moved > 0.25 * scale).all(), f"the oracle's rows do not depend on the needle enough: {moved} of {scale}"
    core = make_core(None, dtype, 16, pages=-(-len(toks) // 16) + 2, seqs=2, model=sized.model(dtype), graphs=True)
    core.start_request("a")
    got = []
    for at in range(0, context + 1, 1024):
        part = toks[at:min(at + 1024, context + 1)]
        last = at + len(part) == context + 1
        out = core.run([StepEntry("a", part, [len(part) - 1] if last else [])])
        if last:
            got.append(out.cpu().numpy())
    for i in range(context + 1, len(toks)):
        out = core.run([StepEntry("a", toks[i:i + 1], [0])]).cpu().numpy()
        if i in rows:
            got.append(out)
    assert core.graph_replays >= 2
    check_logits(dtype, np.concatenate(got), want, scale, f"needle at {place} of {context}")


# ------------------------------------------------------------------ the workloads of the larger configurations
def _follows(sized, prompt, out, dtype, what):
    """Every generated token is the plain implementation's choice given all before it (bfloat16: within 4 % of the
    largest logit of the maximum)."""
    rows = list(range(len(prompt) - 1, len(prompt) + len(out) - 1))
    logits = sized.plain(prompt + out[:-1], rows)
    for k, t in enumerate(out):
        margin = float(logits[k].max() - logits[k][t])
        allowed = (1e-4 if dtype == "float32" else 0.04) * float(np.abs(logits[k]).max())
        assert margin <= allowed, f"{what}, token {k}: engine's {t} is {margin} below the plain maximum"


@pytest.mark.parametrize("dtype,running,longest", [("bfloat16", 32, 4096), ("float32", 8, 1500)])
def test_running_decodes_joined_by_long_prompts_in_portions_with_a_shared_prefix(dtype, running, longest):
    """The continuous-batching mix of the 14B sizes (two layers): requests decoding at contexts drawn from
    [512, longest] are joined by 4 prompts (3,000 tokens, or 1,200 in 32-bit), prefilled in portions of 512 under a
    budget of 2,048 tokens a step beside the decodes; two of the prompts share their first 1,024 tokens, which the
    second one must find in the cache.  Every token of every request against the plain implementation."""
    from jax_vllm_amd.engine.llm import LLM
    from jax_vllm_amd.engine.request import SamplingParams

    sized = Sized(CONFIG_14B, seed=2)
    vocab = sized.cfg.vocab_size
    rng = np.random.default_rng(running)
    join_len = 3000 if dtype == "bfloat16" else 1200
    llm = LLM(sized.model(dtype), dtype=dtype, block_size=16, max_num_seqs=running + 4, max_model_len=longest + 128,
              num_blocks=1 + running * (-(-(longest + 64) // 16)) + 4 * (-(-(join_len + 64) // 16)),
              max_num_batched_tokens=2048, max_chunk=512, enable_prefix_cache=True)
    first = [rng.integers(0, vocab, size=int(n)).tolist() for n in rng.integers(512, longest + 1, size=running)]
    rids = [llm.add_request(p, SamplingParams(max_new_tokens=40)) for p in first]
    outs = {}

    def step():
        for e in llm.step():
            outs.setdefault(e.request_id, []).append(e.token)

    while any(not outs.get(r) for r in rids):
        step()
    for _ in range(4):                       # decode steps of the running requests alone
        step()
    prefix = rng.integers(0, vocab, size=1024).tolist()
    joining = [rng.integers(0, vocab, size=join_len).tolist() for _ in range(4)]
    for p in joining[-2:]:
        p[:1024] = prefix
    hits = llm.stats.cache_hit_tokens
    new = [llm.add_request(p, SamplingParams(max_new_tokens=6)) for p in joining]
    mixed_steps = 0
    while llm.has_work():
        before = llm.stats.prefill_tokens, llm.stats.decode_tokens
        step()
        mixed_steps += llm.stats.prefill_tokens > before[0] and llm.stats.decode_tokens > before[1]
    assert llm.stats.cache_hit_tokens - hits == 1024 and mixed_steps >= 2
    assert llm.stats.max_batched_tokens <= 2048 and llm.stats.graph_replays > 0 and llm.stats.preemptions == 0
    llm.core.cache.check_invariants()
    for i, (p, r) in enumerate(zip(first + joining, rids + new)):
        assert len(outs[r]) == (40 if i < running else 6)
        _follows(sized, p, outs[r], dtype, f"request {i}")


def test_decodes_behind_16k_tokens_at_the_32b_head_geometry():
    """The long-context workload of the 32B sizes (two layers, bfloat16): requests behind prompts of about 16,400
    tokens decode together, their steps recorded and replayed (8 query heads share a kv head, block tables of more
    than a thousand pages).  Every token against the plain implementation."""
    from jax_vllm_amd.engine.llm import LLM
    from jax_vllm_amd.engine.request import SamplingParams

    sized = Sized(CONFIG_32B, seed=3)
    vocab = sized.cfg.vocab_size
    rng = np.random.default_rng(16)
    lens = [16384, 16400, 16385, 16431]
    prompts = [rng.integers(0, vocab, size=n).tolist() for n in lens]
    llm = LLM(sized.model("bfloat16"), dtype="bfloat16", block_size=16, max_num_seqs=4, max_model_len=16512,
              max_num_batched_tokens=2048, enable_prefix_cache=False)
    outs = llm.generate(prompts, SamplingParams(max_new_tokens=10))
    assert llm.stats.graph_replays >= 6 and llm.stats.steps_ahead >= 6
    for i, (p, o) in enumerate(zip(prompts, outs)):
        assert len(o) == 10
        _follows(sized, p, o, "bfloat16", f"request {i}")
