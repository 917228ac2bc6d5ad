"""The engine on the GPU against the plain implementation: generation through the entry
point, scheduling under pressure, graphs, long decoding, first tokens, parts alone, and the
generality of layers (a schedule that repeats a layer and shares a cache, windows, a toy mixer
with state of its own registered from here)."""
import math

import numpy as np
import pytest
import torch

from tests.gpu_util import check_logits, check_tokens_follow, make_core, make_folder, plain_of
from tests.plain import qwen3_plain as P
from tests.tiny import ALL_TINY, TINY_A, TINY_B, TINY_C

pytestmark = pytest.mark.gpu
DTYPES = ["float32", "bfloat16"]


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    return {t["name"]: make_folder(t, tmp_path_factory.mktemp(f"m{t['name']}")) for t in ALL_TINY}


def entry(rid, tokens, want=None):
    from jax_vllm_amd.engine.entries import StepEntry

    return StepEntry(rid, tokens, range(len(tokens)) if want is None else want)


# ------------------------------------------------------------------ generation through the entry point
@pytest.mark.parametrize("dtype", DTYPES)
def test_greedy_generation_workload_a(folders, dtype):
    """Workload A: 3 requests, prompts of 5, 17 and 33 random ids, greedy, 16 new tokens."""
    from jax_vllm_amd import LLM, SamplingParams

    cfg, w = plain_of(folders["A"])
    rng = np.random.default_rng(0)
    prompts = [rng.integers(0, cfg["vocab_size"], size=n).tolist() for n in (5, 17, 33)]
    llm = LLM(folders["A"], dtype=dtype, block_size=TINY_A["page_size"], max_num_seqs=3, max_model_len=64,
              max_num_batched_tokens=32)
    got = llm.generate(prompts, SamplingParams(max_new_tokens=16))
    assert [len(g) for g in got] == [16, 16, 16]
    for p, g in zip(prompts, got):
        check_tokens_follow(dtype, cfg, w, p, g)
    if dtype == "float32":
        assert got == [P.greedy_generate(w, cfg, p, 16) for p in prompts]
    # the reference's functional spelling drives the same engine
    from jax_vllm_amd import add_request, has_work, make_driver, step

    drv = make_driver(folders["A"], max_num_seqs=1, max_model_len=64, block_size=TINY_A["page_size"], dtype=dtype)
    add_request(drv, prompts[1], SamplingParams(max_new_tokens=16))
    out = []
    while has_work(drv):
        out += [ev.token for ev in step(drv)]
    assert out == got[1]


@pytest.mark.parametrize("dtype", ["fp32", "bf16"])
def test_command_line_generates_what_the_plain_implementation_does(folders, dtype, tmp_path, capsys):
    """``main`` from the options to the printed token ids (the reference's entry is
    jllm/server.py:245-306; tokens in, tokens out here): prompts from --prompt-ids and from a
    file, prewarm on (the default), one line of ids per prompt on standard output."""
    from jax_vllm_amd.engine import cli

    cfg, w = plain_of(folders["C"])
    rng = np.random.default_rng(23)
    prompts = [rng.integers(0, cfg["vocab_size"], size=n).tolist() for n in (3, 32, 45)]
    (tmp_path / "p.txt").write_text("\n".join(" ".join(map(str, p)) for p in prompts[1:]) + "\n")
    code = cli.main(["--model-path", str(folders["C"]), "--prompt-ids", ",".join(map(str, prompts[0])),
                     "--prompt-file", str(tmp_path / "p.txt"), "--max-new-tokens", "8", "--dtype", dtype,
                     "--block-size", str(TINY_C["page_size"]), "--max-model-len", "128", "--max-num-seqs", "3",
                     "--max-num-batched-tokens", "40", "--stats"])
    assert code == 0
    cap = capsys.readouterr()
    lines = [l for l in cap.out.splitlines() if l.strip()]
    assert len(lines) == 3 and "prewarmed in" in cap.err and "EngineStats(" in cap.err
    got = [[int(t) for t in l.split()] for l in lines]
    assert [len(g) for g in got] == [8, 8, 8]
    if dtype == "fp32":
        assert got == [P.greedy_generate(w, cfg, p, 8) for p in prompts]
    for p, g in zip(prompts, got):
        check_tokens_follow(dtype, cfg, w, p, g)
    # an eos id ends a request early and is printed
    code = cli.main(["--model-path", str(folders["C"]), "--prompt-ids", " ".join(map(str, prompts[0])), "--max-new-tokens", "8",
                     "--dtype", "fp32", "--block-size", "32", "--max-model-len", "64", "--no-prewarm", "--no-hip-graphs",
                     "--eos-id", str(P.greedy_generate(w, cfg, prompts[0], 8)[2])])
    out = [int(t) for t in capsys.readouterr().out.split()]
    want = P.greedy_generate(w, cfg, prompts[0], 8)
    assert code == 0 and out == want[:want.index(want[2]) + 1]


@pytest.mark.parametrize("dtype", DTYPES)
def test_prewarm_leaves_the_engine_as_it_was(folders, dtype):
    """``prewarm`` (the reference's ``jllm/engine/engine.py:182-208``) captures the decode step for
    every batch bucket and then leaves no trace: request ids start at 0, the counters are zero,
    nothing is in the prefix index, all pages are free, and generation gives the same tokens as
    an engine that was not warmed."""
    from jax_vllm_amd import LLM, SamplingParams, prewarm

    cfg, w = plain_of(folders["B"])
    rng = np.random.default_rng(9)
    prompts = [rng.integers(0, cfg["vocab_size"], size=n).tolist() for n in (3, 20, 41)]
    opts = dict(dtype=dtype, block_size=TINY_B["page_size"], max_num_seqs=5, max_model_len=96, max_num_batched_tokens=64)
    cold = LLM(folders["B"], **opts)
    warm = LLM(folders["B"], **opts)
    pool = warm.core.cache.groups[0].pool
    free = pool.num_free
    seconds = prewarm(warm)
    assert seconds > 0 and not warm.has_work() and warm.requests == {}
    assert warm.stats.steps_run == 0 and warm.stats.emitted_tokens == 0 and warm.stats.admissions == 0
    assert warm.stats.graph_replays == 0
    assert len(warm.core._graphs) >= 3                       # buckets 1, 2, 4 (and 5 rows in the bucket of 8)
    warm.core.cache.check_invariants()
    assert pool.num_free == free and not pool._by_hash       # all pages free, none indexed by content
    assert warm.add_request(prompts[0], SamplingParams(max_new_tokens=2)) == 0
    warm.abort_all()
    sp = SamplingParams(max_new_tokens=12)
    got_warm, got_cold = warm.generate(prompts, sp), cold.generate(prompts, sp)
    assert warm.stats.cache_hit_tokens == 0
    if dtype == "float32":
        assert got_warm == got_cold
    for p, g in zip(prompts, got_warm):
        check_tokens_follow(dtype, cfg, w, p, g)
    with pytest.raises(RuntimeError):
        warm.add_request(prompts[1], sp)
        warm.prewarm()
    warm.abort_all()


@pytest.mark.parametrize("dtype", DTYPES)
def test_request_ids_used_again_after_prewarm_read_their_own_pages(folders, dtype):
    """``prewarm`` gives its warm-up requests the ids 0, 1, ... and hands the same ids to the first
    real requests.  A captured decode step keeps a copy of every row's block table and rewrites
    it only when the table's signature changes; a real request whose table has the same number of
    reserves as the warm-up request of the same id (a prompt of exactly one or two pages; a
    prompt cut into two portions by the token budget) must still get its own pages into the row.
    The pool is drawn on first, so the real requests' pages are not the warm-up's."""
    from jax_vllm_amd import LLM, SamplingParams

    cfg, w = plain_of(folders["B"])
    ps = TINY_B["page_size"]
    rng = np.random.default_rng(31)
    opts = dict(dtype=dtype, block_size=ps, max_num_seqs=4, max_model_len=160, max_num_batched_tokens=64,
                enable_prefix_cache=False)
    for lengths in ([ps, 2 * ps, 3 * ps], [100, ps]):          # 100 tokens under a budget of 64: two portions
        llm = LLM(folders["B"], **opts)
        llm.prewarm()
        # hold a few pages so that the next requests get other pages than the warm-up requests had
        held = [llm.core.cache.groups[0].pool.allocate() for _ in range(7)]
        prompts = [rng.integers(0, cfg["vocab_size"], size=n).tolist() for n in lengths]
        got = llm.generate(prompts, SamplingParams(max_new_tokens=10))
        assert llm.stats.graph_replays > 0
        for p, g in zip(prompts, got):
            check_tokens_follow(dtype, cfg, w, p, g)
        llm.core.cache.groups[0].pool.release(held)
        llm.core.cache.check_invariants()


def test_temperature_generation_workload_b_is_cut_independent(folders):
    """Workload B: prompts 1/9/40/64/100 (two share a 32-token prefix), arrivals at steps
    0,0,2,3,5, budget 24, temperature 0.8, seed 7, 20 new tokens.  The draws are keyed by
    (seed, request, index), so another budget, batch width or page pool gives the same tokens."""
    from jax_vllm_amd import LLM, SamplingParams

    cfg, w = plain_of(folders["B"])
    rng = np.random.default_rng(1)
    shared = rng.integers(0, cfg["vocab_size"], size=32).tolist()
    prompts = [rng.integers(0, cfg["vocab_size"], size=1).tolist(), rng.integers(0, cfg["vocab_size"], size=9).tolist(),
               shared + rng.integers(0, cfg["vocab_size"], size=8).tolist(),
               shared + rng.integers(0, cfg["vocab_size"], size=32).tolist(),
               rng.integers(0, cfg["vocab_size"], size=100).tolist()]
    sp = SamplingParams(max_new_tokens=20, temperature=0.8, seed=7)
    base = dict(dtype="fp32", block_size=16, max_model_len=128)
    a = LLM(folders["B"], max_num_seqs=4, max_num_batched_tokens=24, **base)
    got = a.generate(prompts, sp, arrival_steps=[0, 0, 2, 3, 5])
    assert a.stats.cache_hit_blocks >= 1 and a.stats.max_batched_tokens <= 24
    b = LLM(folders["B"], max_num_seqs=1, max_num_batched_tokens=2048, enable_prefix_cache=False, **base)
    assert b.generate(prompts, sp) == got
    c = LLM(folders["B"], max_num_seqs=3, max_num_batched_tokens=7, num_blocks=1 + 9, **base)
    assert c.generate(prompts, sp) == got
    # not simply greedy; and each token is the one that the same draw picks from the *plain*
    # logits: the draw of request r's i-th token has the key of (seed, r, i) and depends on nothing
    # else, so the sampling kernel applied to the plain implementation's last row must give the
    # engine's token (that the kernel's draws follow softmax(logits / T) is the kernel tests' subject)
    from jax_vllm_amd.ops import kernels as K
    from jax_vllm_amd.sampling import draw_key

    greedy = LLM(folders["B"], max_num_seqs=4, max_num_batched_tokens=2048, **base).generate(prompts, SamplingParams(max_new_tokens=20))
    assert greedy != got
    rows, keys, flat = [], [], []
    for r, (p, g) in enumerate(zip(prompts, got)):
        seq = list(p)
        for i, t in enumerate(g):
            rows.append(P.forward(w, cfg, seq)[-1])
            keys.append(draw_key(7, r, i))
            flat.append(t)
            seq.append(t)
    picked = K.sample(torch.stack(rows).cuda(), torch.full((len(rows),), 0.8, device="cuda"),
                      torch.tensor(keys, dtype=torch.int64, device="cuda")).tolist()
    assert picked == flat


@pytest.mark.parametrize("dtype", DTYPES)
def test_few_pages_preemption_and_prefix_reuse_give_the_same_tokens(folders, dtype):
    from jax_vllm_amd import LLM, SamplingParams

    cfg, w = plain_of(folders["C"])
    rng = np.random.default_rng(2)
    # every request fits when admitted and grows into one more page while decoding
    prompts = [rng.integers(0, cfg["vocab_size"], size=n).tolist() for n in (60, 62, 30, 28)]
    sp = SamplingParams(max_new_tokens=24)
    roomy = LLM(folders["C"], dtype=dtype, block_size=32, max_num_seqs=4, max_model_len=128, max_num_batched_tokens=512,
                enable_prefix_cache=False, use_hip_graphs=False)
    want = roomy.generate(prompts, sp)
    tight = LLM(folders["C"], dtype=dtype, block_size=32, max_num_seqs=4, max_model_len=128, max_num_batched_tokens=48,
                num_blocks=1 + 6)
    got = tight.generate(prompts, sp)
    assert tight.stats.preemptions > 0
    if dtype == "float32":
        assert got == want
    for p, g in zip(prompts, got):
        check_tokens_follow(dtype, cfg, w, p, g)
    tight.core.cache.check_invariants()
    # with room to keep them, full pages of a prompt seen before are found in the cache
    keep = LLM(folders["C"], dtype=dtype, block_size=32, max_num_seqs=2, max_model_len=128, max_num_batched_tokens=48,
               num_blocks=1 + 12)
    first = keep.generate(prompts[:2], sp)
    again = keep.generate(prompts[:2], sp)
    assert keep.stats.cache_hit_blocks == 2 and keep.stats.cache_hit_tokens == 64
    if dtype == "float32":
        assert first == again == want[:2]
    for p, g in zip(prompts[:2], again):
        check_tokens_follow(dtype, cfg, w, p, g)


@pytest.mark.parametrize("dtype", DTYPES)
def test_replayed_decode_steps_equal_eager_steps(folders, dtype):
    """A captured decode step is replayed several times with eager work (prompt portions, other
    batch widths) in between; every replay must give what the eager launches give."""
    cfg, w = plain_of(folders["B"])
    rng = np.random.default_rng(3)
    reqs = {f"r{i}": rng.integers(0, cfg["vocab_size"], size=n).tolist() for i, n in enumerate((60, 41, 75))}
    eager = make_core(folders["B"], dtype, 16, graphs=False)
    graph = make_core(folders["B"], dtype, 16, graphs=True, model=eager.model)
    for core in (eager, graph):
        for rid in reqs:
            core.start_request(rid)
    outs = {id(eager): [], id(graph): []}
    for core in (eager, graph):
        core.run([entry(r, t[:20], []) for r, t in reqs.items()])
        for i in range(20, 40):
            live = [r for r, t in reqs.items() if i < len(t)]
            outs[id(core)].append(core.run([entry(r, reqs[r][i:i + 1], [0]) for r in live]).cpu())
            if i == 30:   # eager work between replays: a prompt portion of a new request, then its end
                core.start_request("x")
                core.run([entry("x", reqs["r0"][:13], [12])])
                core.finish_request("x")
    assert graph.graph_replays >= 15 and eager.graph_replays == 0
    for a, b in zip(outs[id(eager)], outs[id(graph)]):
        torch.testing.assert_close(a, b, rtol=0, atol=0)
    expected = {r: P.forward(w, cfg, t).numpy() for r, t in reqs.items()}
    for i, got in zip(range(20, 40), outs[id(graph)]):
        live = [r for r, t in reqs.items() if i < len(t)]
        check_logits(dtype, got.numpy(), np.stack([expected[r][i] for r in live]), what=f"position {i}")


@pytest.mark.parametrize("dtype", DTYPES)
def test_decode_steps_started_ahead_give_the_same_tokens(folders, dtype):
    """With ``decode_ahead`` a captured decode step is started before the tokens of the step before
    it are on the host (it takes them from the sampling output on the device).  Greedy and drawn
    tokens, requests that end on an eos_id in the middle of that (one row of the step under way is
    then for nothing), requests that join later and prefixes taken from the cache: the tokens are
    those of an engine that waits for every step, and those of the plain implementation."""
    from jax_vllm_amd import LLM, SamplingParams

    cfg, w = plain_of(folders["B"])
    rng = np.random.default_rng(17)
    shared = rng.integers(0, cfg["vocab_size"], size=40).tolist()
    prompts = [rng.integers(0, cfg["vocab_size"], size=n).tolist() for n in (9, 33, 18)] + [shared + [3, 4], shared + [5]]
    plain = [P.greedy_generate(w, cfg, p, 24) for p in prompts]
    params = [SamplingParams(max_new_tokens=24), SamplingParams(max_new_tokens=24, eos_id=plain[1][7]),
              SamplingParams(max_new_tokens=17, temperature=0.8, seed=5), SamplingParams(max_new_tokens=24),
              SamplingParams(max_new_tokens=20, eos_id=plain[4][11])]
    outs = {}
    for ahead in (False, True):
        llm = LLM(folders["B"], dtype=dtype, block_size=16, max_num_seqs=5, max_model_len=128,
                  max_num_batched_tokens=64, decode_ahead=ahead)
        got = {}
        rids = [llm.add_request(p, sp) for p, sp in zip(prompts[:3], params[:3])]
        calls = 0
        while llm.has_work():
            for ev in llm.step():
                got.setdefault(ev.request_id, []).append(ev.token)
            calls += 1
            if calls in (6, 13):          # two requests join while decode steps follow each other
                rids.append(llm.add_request(prompts[len(rids)], params[len(rids)]))
        outs[ahead] = [got[r] for r in rids]
        assert (llm.core.steps_followed > 10) == ahead and llm.core.graph_replays > 10
        llm.core.cache.check_invariants()
        assert llm.core.cache.num_free_pages() == llm.config.usable_pages and not llm.core.cache.requests
        assert llm.stats.cache_hit_tokens >= 32
        again = llm.generate(prompts[:2], params[:2])             # the engine is as good as new afterwards
        assert again == outs[ahead][:2]
    assert outs[True] == outs[False]
    for i in (0, 1, 3, 4):                                        # the greedy ones against the plain implementation
        got = outs[True][i]
        eos = params[i].eos_id
        if dtype == "float32":
            want = plain[i][:plain[i].index(eos) + 1] if eos is not None and eos in plain[i] else plain[i][:params[i].max_new_tokens]
            assert got == want
        else:
            check_tokens_follow(dtype, cfg, w, prompts[i], got)
    assert len(outs[True][2]) == 17


@pytest.mark.parametrize("dtype", DTYPES)
def test_replayed_decode_steps_of_many_requests(folders, dtype):
    """Captured decode steps with 20 and then 40 live requests (rows of the step: 24 and 48, of
    which the last are padding), while requests end and the rows are handed to others: every
    row's logits against the plain implementation.  The replays' padding rows read the null page
    and store nothing."""
    cfg, w = plain_of(folders["B"])
    rng = np.random.default_rng(17)
    lengths = [int(n) for n in rng.integers(20, 56, size=40)]
    reqs = {f"r{i}": rng.integers(0, cfg["vocab_size"], size=n).tolist() for i, n in enumerate(lengths)}
    expected = {r: P.forward(w, cfg, t).numpy() for r, t in reqs.items()}
    core = make_core(folders["B"], dtype, 16, pages=200, seqs=48, graphs=True)
    fed = {}

    def admit(names, first):
        for r in names:
            core.start_request(r)
            fed[r] = first
        core.run([entry(r, reqs[r][:first], []) for r in names])

    def decode_all():
        live = [r for r in fed if fed[r] < len(reqs[r])]
        out = core.run([entry(r, reqs[r][fed[r]:fed[r] + 1], [0]) for r in live]).cpu().numpy()
        check_logits(dtype, out, np.stack([expected[r][fed[r]] for r in live]), what=f"{len(live)} live")
        for r in live:
            fed[r] += 1
            if fed[r] == len(reqs[r]):
                core.finish_request(r)
        return len(live)

    names = list(reqs)
    admit(names[:20], 12)
    widths = [decode_all() for _ in range(6)]
    assert widths == [20] * 6
    admit(names[20:], 15)
    while any(fed[r] < len(reqs[r]) for r in fed):
        widths.append(decode_all())
    assert 40 in widths and any(17 <= x <= 24 for x in widths[6:])    # rows of 48 and of 24, rows handed on
    assert {k[0] for k in core._graphs} >= {24, 48} and core.graph_replays >= 20
    core.cache.check_invariants()
    assert core.cache.num_free_pages() == 200


@pytest.mark.parametrize("dtype", DTYPES)
def test_replayed_decode_steps_with_a_window_group(folders, dtype):
    """A model with a full-attention layer group and a windowed one, decoded through captured
    steps: the window group's table rows change as pages are given back (its signature moves,
    the captured step's copy of the row must follow)."""
    cfg, w = plain_of(folders["B"])
    schedule = [(0, None), (1, None), (2, None)]
    windows = {1: 20}
    model = custom_model(folders["B"], dtype, schedule, windows)
    core = make_core(None, dtype, 16, pages=30, seqs=3, model=model, graphs=True)
    assert core.group_keys == [("full",), ("window", 20)]
    rng = np.random.default_rng(19)
    reqs = {r: rng.integers(0, cfg["vocab_size"], size=n).tolist() for r, n in (("a", 120), ("b", 90))}
    want = {r: P.forward_scheduled(w, cfg, t, schedule, windows).numpy() for r, t in reqs.items()}
    got = {r: [] for r in reqs}
    for r in reqs:
        core.start_request(r)
    out = core.run([entry("a", reqs["a"][:30]), entry("b", reqs["b"][:7])]).cpu().numpy()
    got["a"].append(out[:30]), got["b"].append(out[30:])
    fed = {"a": 30, "b": 7}
    while any(fed[r] < len(reqs[r]) for r in reqs):
        live = [r for r in reqs if fed[r] < len(reqs[r])]
        out = core.run([entry(r, reqs[r][fed[r]:fed[r] + 1]) for r in live]).cpu().numpy()
        for i, r in enumerate(live):
            got[r].append(out[i:i + 1])
            fed[r] += 1
    assert core.graph_replays >= 80
    for r in reqs:
        check_logits(dtype, np.concatenate(got[r]), want[r], what=r)
    assert core.cache.block_table("a", 1)[:5] == [0] * 5        # the window has moved on


# ------------------------------------------------------------------ long decoding, first tokens
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("graphs", [False, True])
def test_long_decoding(folders, dtype, graphs):
    cfg, w = plain_of(folders["A"])
    toks = np.random.default_rng(4).integers(0, cfg["vocab_size"], size=300).tolist()
    want = P.forward(w, cfg, toks).numpy()
    core = make_core(folders["A"], dtype, TINY_A["page_size"], pages=40, graphs=graphs)
    core.start_request("a")
    got = [core.run([entry("a", toks[:9])]).cpu().numpy()]
    for i in range(9, 300):
        got.append(core.run([entry("a", toks[i:i + 1])]).cpu().numpy())
    check_logits(dtype, np.concatenate(got), want)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("tiny", ALL_TINY, ids=[t["name"] for t in ALL_TINY])
def test_first_tokens_of_a_sequence(folders, dtype, tiny):
    cfg, w = plain_of(folders[tiny["name"]])
    toks = [7, 3, 11, 2, 5]
    want = P.forward(w, cfg, toks).numpy()
    core = make_core(folders[tiny["name"]], dtype, tiny["page_size"])
    for rid, cuts in (("one", [1, 1, 1, 1, 1]), ("two", [1, 2, 2]), ("whole", [5])):
        core.start_request(rid)
        got, at = [], 0
        for n in cuts:
            got.append(core.run([entry(rid, toks[at:at + n])]).cpu().numpy())
            at += n
        check_logits(dtype, np.concatenate(got), want, what=rid)


def _drawn_config(seed: int) -> dict:
    """A configuration drawn from everything config.json allows: any group ratio, head sizes in
    steps of 16 and a few that are only even, widths that are no multiple of 4, 8, 16 or 64, tied or
    untied heads, feed-forward widths whose 512-column phases share out unevenly."""
    rng = np.random.default_rng(seed)
    nkv = int(rng.choice([1, 2, 3, 4]))
    nq = nkv * int(rng.choice([1, 2, 3, 4, 8]))
    d = int(rng.choice([16, 32, 48, 64, 80, 96, 128, 144, 256, 24, 40]))
    hidden = int(rng.choice([6, 8, 24, 40, 50, 64, 100, 136, 256, 520, 1024]))
    inter = int(rng.choice([16, 18, 50, 56, 72, 256, 1000, 1536, 3072, 6152]))
    return dict(
        name=f"drawn{seed}", seed=seed, std=0.08, norm_std=0.1, page_size=int(rng.choice([8, 16, 32, 64])),
        config=dict(architectures=["Qwen3ForCausalLM"], num_hidden_layers=int(rng.choice([1, 2])), hidden_size=hidden,
                    num_attention_heads=nq, num_key_value_heads=nkv, head_dim=d, intermediate_size=inter,
                    vocab_size=int(rng.choice([50, 257, 1000, 4099])), rope_theta=float(rng.choice([1e4, 1e6])),
                    rms_norm_eps=float(rng.choice([1e-6, 1e-5])), tie_word_embeddings=bool(rng.integers(2)),
                    max_position_embeddings=4096))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("seed", range(20))
def test_drawn_configurations(tmp_path, dtype, seed):
    """Twenty drawn configurations: a prompt whole, one in two portions beside it, then both decoded
    with 18 further requests of one token beside them (so the step has 20 rows: the matrix products
    for 17..64 rows), everything against the plain implementation.  No size may be refused."""
    tiny = _drawn_config(seed)
    folder = make_folder(tiny, tmp_path)
    cfg, w = plain_of(folder)
    rng = np.random.default_rng(100 + seed)
    ps = tiny["page_size"]
    a = rng.integers(0, cfg["vocab_size"], size=41).tolist()
    b = rng.integers(0, cfg["vocab_size"], size=37).tolist()
    want_a, want_b = P.forward(w, cfg, a).numpy(), P.forward(w, cfg, b).numpy()
    core = make_core(folder, dtype, ps, pages=20 * (-(-64 // ps)) + 4, seqs=20)
    scale = max(float(np.abs(want_a).max()), float(np.abs(want_b).max()))
    core.start_request("a")
    core.start_request("b")
    got = core.run([entry("a", a[:30]), entry("b", b[:9])]).cpu().numpy()
    check_logits(dtype, got[:30], want_a[:30], scale, "a whole")
    check_logits(dtype, got[30:], want_b[:9], scale, "b first portion")
    got = core.run([entry("b", b[9:33])]).cpu().numpy()
    check_logits(dtype, got, want_b[9:33], scale, "b second portion")
    others = [f"o{i}" for i in range(18)]
    for r in others:
        core.start_request(r)
    fed_a, fed_b = 30, 33
    for step in range(4):
        entries = [entry("a", a[fed_a:fed_a + 1]), entry("b", b[fed_b:fed_b + 1])]
        entries += [entry(r, [int(rng.integers(0, cfg["vocab_size"]))], []) for r in others]
        got = core.run(entries).cpu().numpy()
        check_logits(dtype, got[0], want_a[fed_a], scale, f"a decoded {step}")
        check_logits(dtype, got[1], want_b[fed_b], scale, f"b decoded {step}")
        fed_a, fed_b = fed_a + 1, fed_b + 1
    for r in ["a", "b"] + others:
        core.finish_request(r)
    core.cache.check_invariants()


def test_step_function_refuses_bad_input(folders):
    from jax_vllm_amd.cache import OutOfPages

    core = make_core(folders["A"], "float32", 8, pages=2)
    core.start_request("a")
    with pytest.raises(ValueError, match="outside the vocabulary"):
        core.run([entry("a", [256])])
    with pytest.raises(ValueError, match="wanted place"):
        core.run([entry("a", [1, 2], [2])])
    with pytest.raises(OutOfPages):
        core.run([entry("a", list(range(17)))])
    assert core.run([entry("a", list(range(16)), [15])]).shape == (1, 256)   # nothing was consumed by the refusals
    core.cache.check_invariants()
    # a step whose second entry has no room leaves the first entry's table as it was
    core = make_core(folders["A"], "float32", 8, pages=3)
    core.start_request("a"), core.start_request("b")
    core.run([entry("a", [1, 2, 3], [])])
    with pytest.raises(OutOfPages, match="'b'"):
        core.run([entry("a", list(range(8))), entry("b", list(range(9)))])      # 2 pages for a, 2 for b, 3 in the pool
    assert len(core.cache.block_table("a", 0)) == 1 and core.cache.block_table("b", 0) == []
    assert core.cache.num_free_pages() == 2
    assert core.run([entry("a", list(range(8)), [7]), entry("b", [5], [0])]).shape == (2, 256)
    core.cache.check_invariants()


# ------------------------------------------------------------------ each part alone
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_parts_alone(dtype):
    from jax_vllm_amd.parts import PartSpec, build_part

    g = torch.Generator().manual_seed(11)
    tol = dict(rtol=1e-5, atol=1e-5) if dtype == torch.float32 else dict(rtol=3e-2, atol=3e-2)
    hidden, inter, vocab, t = 72, 200, 333, 9
    x = torch.randn(t, hidden, generator=g)

    norm = build_part("norm", PartSpec("rmsnorm", {"size": hidden, "eps": 1e-4}))
    wn = 1 + 0.2 * torch.randn(hidden, generator=g)
    norm.bind({"weight": wn.cuda()}, dtype)
    h = x.clone().cuda()
    delta = torch.randn(t, hidden, generator=g).to(dtype)
    out = norm.add_norm(h, delta.cuda())
    torch.testing.assert_close(h.cpu(), x + delta.float())
    torch.testing.assert_close(out.float().cpu(), P.rms_norm(wn, 1e-4, x + delta.float()), **tol)
    # the delta as a stack of float partial products: added in order, then to the residual
    h3 = x.clone().cuda()
    parts = torch.randn(3, t, hidden, generator=g)
    out3 = norm.add_norm(h3, parts.cuda())
    total = (parts[0] + parts[1]) + parts[2]
    torch.testing.assert_close(h3.cpu(), x + total, rtol=0, atol=0)
    torch.testing.assert_close(out3.float().cpu(), P.rms_norm(wn, 1e-4, x + total), **tol)
    rows = torch.tensor([4, 0], dtype=torch.int32).cuda()
    out_rows = norm.add_norm(h3, parts.cuda(), rows=rows)   # selected rows only, h untouched
    torch.testing.assert_close(h3.cpu(), x + total, rtol=0, atol=0)
    torch.testing.assert_close(out_rows.float().cpu(), P.rms_norm(wn, 1e-4, (x + total + total)[[4, 0]]), **tol)
    torch.testing.assert_close(norm.forward(x.to(dtype).cuda()).float().cpu(), P.rms_norm(wn, 1e-4, x.to(dtype).float()), **tol)

    mlp = build_part("feed_forward", PartSpec("gated_mlp", {"hidden_size": hidden, "intermediate_size": inter}))
    ws = {k: (0.1 * torch.randn(s, generator=g)).to(dtype) for k, s in
          (("gate_proj.weight", (inter, hidden)), ("up_proj.weight", (inter, hidden)), ("down_proj.weight", (hidden, inter)))}
    mlp.bind({k: v.cuda() for k, v in ws.items()}, dtype)
    for rows in (t, 70):   # few rows (streaming kernel) and many (library product)
        xi = torch.randn(rows, hidden, generator=g).to(dtype)
        ref = P.swiglu(ws["gate_proj.weight"].float(), ws["up_proj.weight"].float(), ws["down_proj.weight"].float(), xi.float())
        got = mlp.forward(xi.cuda())
        if got.dim() == 3:                     # a stack of float partial products, added by the next norm
            assert got.dtype == torch.float32
            got = got.sum(0)
        torch.testing.assert_close(got.float().cpu(), ref, **tol)
    # the gate's activation is a parameter of the part: the tanh form of gelu against the library's
    gelu = build_part("feed_forward", PartSpec("gated_mlp", {"hidden_size": hidden, "intermediate_size": inter,
                                                            "activation": "gelu_tanh"}))
    gelu.bind({k: v.cuda() for k, v in ws.items()}, dtype)
    for rows in (t, 40, 70):   # epilogue of the streaming kernels, of the 64-row tiles, kernel after the library
        xi = torch.randn(rows, hidden, generator=g).to(dtype)
        gate = torch.nn.functional.gelu(xi.float() @ ws["gate_proj.weight"].float().T, approximate="tanh")
        ref = (gate * (xi.float() @ ws["up_proj.weight"].float().T)) @ ws["down_proj.weight"].float().T
        got = gelu.forward(xi.cuda())
        got = got.sum(0) if got.dim() == 3 else got
        torch.testing.assert_close(got.float().cpu(), ref, **tol)
    with pytest.raises(ValueError, match="gelu_tanh"):
        build_part("feed_forward", PartSpec("gated_mlp", {"hidden_size": hidden, "intermediate_size": inter,
                                                          "activation": "relu"}))

    emb = build_part("embedding", PartSpec("token_embedding", {"vocab_size": vocab, "hidden_size": hidden}))
    table = torch.randn(vocab, hidden, generator=g).to(dtype)
    emb.bind({"weight": table.cuda()}, dtype)
    ids = torch.tensor([0, 332, 17], dtype=torch.int32)
    torch.testing.assert_close(emb.forward(ids.cuda()).cpu(), P.embed(table.float(), ids.long()))

    head = build_part("head", PartSpec("linear_head", {"vocab_size": vocab, "hidden_size": hidden}))
    head.bind({"weight": table.cuda()}, dtype)
    xi = torch.randn(5, hidden, generator=g).to(dtype)
    logits = head.forward(xi.cuda())
    assert logits.dtype == torch.float32
    torch.testing.assert_close(logits.cpu(), P.linear(table.float(), xi.float()), **tol)

    rot = build_part("position", PartSpec("rotary", {"head_dim": 48, "theta": 5e5}))
    ref_inv = 1.0 / (5e5 ** (torch.arange(0, 48, 2, dtype=torch.float32) / 48))
    torch.testing.assert_close(rot.inverse_frequencies(), ref_inv, rtol=0, atol=0)
    with pytest.raises(ValueError, match="rotary_dim"):
        build_part("position", PartSpec("rotary", {"head_dim": 48, "theta": 1e4, "rotary_dim": 50}))
    with pytest.raises(ValueError, match="no mixer part named"):
        build_part("mixer", PartSpec("nonexistent", {}))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("biased", [False, True])
def test_attention_part_alone(folders, dtype, biased):
    """The mixer with its cache, outside any model: two portions of one request and a second
    request beside it, against the plain attention block.  ``biased``: the part's options
    ``qkv_bias`` and ``o_bias``; a bias is one more input column that is always 1, so the plain
    block gives the reference with the bias as a last column of its weight."""
    from jax_vllm_amd.cache import CacheManager
    from jax_vllm_amd.cache.storage import allocate_memories
    from jax_vllm_amd.parts import PartSpec, build_part, kv_cache_spec
    from jax_vllm_amd.parts.model import RunMemoryPlan
    from jax_vllm_amd.parts.spec import StepContext

    tdt = torch.float32 if dtype == "float32" else torch.bfloat16
    hidden, nq, nkv, d, ps = 80, 6, 3, 32, 8
    g = torch.Generator().manual_seed(12)
    att = build_part("mixer", PartSpec("gqa_attention", dict(
        hidden_size=hidden, num_heads=nq, num_kv_heads=nkv, head_dim=d, qk_norm_eps=1e-5,
        position=PartSpec("rotary", {"head_dim": d, "theta": 1e4}), qkv_bias=biased, o_bias=biased)))
    assert ("q_proj.bias" in att.tensors()) == biased and ("o_proj.bias" in att.tensors()) == biased
    ws = {n: ((0.15 * torch.randn(s.shape, generator=g)) if s.role == "matrix" else
              0.3 * torch.randn(s.shape, generator=g) if n.endswith(".bias") else 1 + 0.1 * torch.randn(s.shape, generator=g))
          for n, s in att.tensors().items()}
    ws = {n: v.to(tdt).float() for n, v in ws.items()}
    att.bind({n: v.to(tdt if att.tensors()[n].role == "matrix" else torch.float32).cuda() for n, v in ws.items()}, tdt)
    plan = [RunMemoryPlan(0, 0, att.cache_spec(), None, None)]
    assert att.cache_spec() == kv_cache_spec(nkv, d, None)
    assert [(t.name, t.page_shape(ps)) for t in att.cache_spec().tensors] == [("k", (nkv, ps, d)), ("v", (nkv, d, ps))]
    mem = allocate_memories(plan, [("full",)], 16, ps, 2, tdt, "cuda")[0]
    cache = CacheManager([("full",)], ps, 16, 2, enable_prefix_cache=False)
    cfg = dict(num_heads=nq, num_kv_heads=nkv, head_dim=d, rms_norm_eps=1e-5, rope_theta=1e4)
    xa, xb = torch.randn(21, hidden, generator=g).to(tdt), torch.randn(5, hidden, generator=g).to(tdt)
    pw = {f"p.{n}": v for n, v in ws.items()}
    one = lambda x: x.float()
    if biased:
        for n in ("q_proj", "k_proj", "v_proj"):
            pw[f"p.{n}.weight"] = torch.cat([ws[f"{n}.weight"], ws[f"{n}.bias"][:, None]], dim=1)
        one = lambda x: torch.cat([x.float(), torch.ones(x.shape[0], 1)], dim=1)
    want_a = P.attention_block(pw, "p", cfg, one(xa), torch.arange(21))
    want_b = P.attention_block(pw, "p", cfg, one(xb), torch.arange(5))
    if biased:
        want_a, want_b = want_a + ws["o_proj.bias"], want_b + ws["o_proj.bias"]
    cache.start("a"), cache.start("b")

    def step(parts):
        q_lens = [x.shape[0] for _, x in parts]
        ctxl = [cache.context_len(r) for r, _ in parts]
        for (r, x) in parts:
            cache.reserve(r, x.shape[0])
        i32 = lambda v: torch.tensor(v, dtype=torch.int32).cuda()
        width = max(len(cache.block_table(r, 0)) for r, _ in parts)
        ctx = StepContext(
            num_tokens=sum(q_lens), num_requests=len(parts),
            positions=i32([c + i for c, q in zip(ctxl, q_lens) for i in range(q)]),
            token_req=i32([j for j, q in enumerate(q_lens) for _ in range(q)]),
            cu_seqlens=i32(np.concatenate([[0], np.cumsum(q_lens)]).tolist()), context_lens=i32(ctxl),
            slot_ids=i32([cache.slot(r) for r, _ in parts]),
            block_tables=[i32([cache.block_table(r, 0) + [0] * (width - len(cache.block_table(r, 0))) for r, _ in parts])],
            slot_mappings=[i32([s for r, x in parts for s in cache.slot_mapping(r, 0, x.shape[0])])],
            page_size=ps, q_lens_host=q_lens, context_lens_host=ctxl, slot_ids_host=[0] * len(parts),
            max_q_len=max(q_lens), max_kv_len=max(c + q for c, q in zip(ctxl, q_lens)))
        out = att.forward(torch.cat([x for _, x in parts]).cuda(), ctx, mem)
        for r, x in parts:
            cache.commit(r, [0] * x.shape[0])
        if out.dim() == 3:                     # float partial products of the output projection
            out = out.sum(0)
        return out.float().cpu()

    tol = dict(rtol=2e-5, atol=2e-5) if dtype == "float32" else dict(rtol=3e-2, atol=3e-2)
    o1 = step([("a", xa[:13])])
    o2 = step([("b", xb), ("a", xa[13:20])])
    o3 = step([("a", xa[20:21])])
    torch.testing.assert_close(torch.cat([o1, o2[5:], o3]), want_a, **tol)
    torch.testing.assert_close(o2[:5], want_b, **tol)


# ------------------------------------------------------------------ layers as data
def custom_model(folder, dtype, schedule, windows):
    """The tiny model's weights under another ModelSpec: the schedule names layers as it likes
    and some layers get an attention window."""
    from jax_vllm_amd.config import resolve
    from jax_vllm_amd.parts import DecoderModel, LayerRun, ModelSpec, PartSpec
    from jax_vllm_amd.weights.loader import TORCH_DTYPES, target_dtype
    from jax_vllm_amd.weights.safetensors_io import SafetensorsFile

    arch, cfg, _ = resolve(folder)
    spec = arch.build_spec(cfg)
    layers = []
    for i, ls in enumerate(spec.layers):
        if i in windows:
            params = dict(ls.mixer.params, window=windows[i])
            ls = type(ls)(**{**{f: getattr(ls, f) for f in ls.__dataclass_fields__}, "mixer": PartSpec(ls.mixer.kind, params)})
        layers.append(ls)
    kw = {f: getattr(spec, f) for f in spec.__dataclass_fields__}
    model = DecoderModel(ModelSpec(**dict(kw, layers=layers, schedule=[LayerRun(l, c) for l, c in schedule])))
    f = SafetensorsFile(folder / "model.safetensors")
    compute = TORCH_DTYPES[dtype]
    model.bind({n: f.tensor(n).cuda().to(target_dtype(ts.role, compute)) for n, ts in model.tensor_specs().items()}, compute)
    return model


@pytest.mark.parametrize("dtype", DTYPES)
def test_schedule_repeats_a_layer_shares_a_cache_and_windows(folders, dtype):
    cfg, w = plain_of(folders["B"])
    schedule = [(0, None), (1, None), (0, None), (2, 0), (1, None)]   # layer 0 and 1 twice; run 3 reads run 0's cache
    windows = {1: 24}
    model = custom_model(folders["B"], dtype, schedule, windows)
    plan = model.memory_plan()
    assert [p.cache_of for p in plan] == [None, None, None, 0, None]
    with pytest.raises(ValueError, match="already given back"):      # all keys wanted of a cache that keeps a window
        make_core(None, dtype, 16, pages=4, model=custom_model(folders["B"], dtype, [(0, None), (1, None), (2, 1)], windows))
    core = make_core(None, dtype, 16, pages=24, model=model)
    assert core.group_keys == [("full",), ("window", 24)]
    toks = np.random.default_rng(5).integers(0, cfg["vocab_size"], size=150).tolist()
    want = P.forward_scheduled(w, cfg, toks, schedule, windows).numpy()
    assert not np.allclose(want, P.forward(w, cfg, toks).numpy(), atol=1e-2)
    core.start_request("a")
    got, at = [], 0
    for n in [31, 2, 40, 1, 1, 17, 50, 3, 5]:
        got.append(core.run([entry("a", toks[at:at + n])]).cpu().numpy())
        at += n
        core.cache.check_invariants()
    assert at == 150
    check_logits(dtype, np.concatenate(got), want)
    # the window group has given pages back, the full group has not
    assert core.cache.block_table("a", 1)[:6] == [0] * 6 and all(core.cache.block_table("a", 0))
    core.finish_request("a")
    assert core.cache.num_free_pages(0) == core.cache.num_free_pages(1) == 24


class RunningMeanMixer:
    """A toy token mixer with state of its own, defined here and registered from here: its
    output at a token is a projection of the mean of all inputs of the request up to and
    including that token.  State per request: the running sum (float).  No pages.  It plans on
    the host (reads the context's host mirrors) and says nothing about replaying, so the engine
    never records its steps."""

    def __init__(self, hidden_size: int):
        self.hidden_size = hidden_size

    def tensors(self):
        from jax_vllm_amd.parts import TensorSpec

        return {"proj.weight": TensorSpec((self.hidden_size, self.hidden_size))}

    def cache_spec(self):
        return None

    def state_spec(self):
        from jax_vllm_amd.parts import StateSpec

        return StateSpec((self.hidden_size,), "float32")

    def bind(self, tensors, dtype):
        self.w = tensors["proj.weight"]

    def forward(self, x, ctx, mem):
        out = torch.empty_like(x)
        at = 0
        for q, c, slot in zip(ctx.q_lens_host, ctx.context_lens_host, ctx.slot_ids_host):
            xs = x[at:at + q].float()
            sums = mem.state[slot][None, :] + torch.cumsum(xs, dim=0)
            mem.state[slot] = sums[-1]
            counts = torch.arange(c + 1, c + q + 1, device=x.device, dtype=torch.float32)[:, None]
            out[at:at + q] = ((sums / counts).to(x.dtype) @ self.w.t()).to(x.dtype)
            at += q
        return out


class RunningMeanMixerOnDevice(RunningMeanMixer):
    """The same function, but a step of single tokens takes slots and positions from the
    context's device tensors only, so it may be recorded and replayed: it declares so."""

    replayable = True

    def forward(self, x, ctx, mem):
        if not ctx.decode_only:
            assert not ctx.captured
            return super().forward(x, ctx, mem)
        slots = ctx.slot_ids.long()
        sums = mem.state[slots] + x.float()
        mem.state[slots] = sums                  # rows that pad a recorded step write the spare row
        counts = (ctx.positions + 1).float()[:, None]
        return ((sums / counts).to(x.dtype) @ self.w.t()).to(x.dtype)


def toy_state_model(dtype, mixer_kind):
    """(bound model, float weights by name) of a four-run model: toy mixer, attention, toy mixer,
    and the first layer once more (its weights shared, a state of its own)."""
    from jax_vllm_amd.config import register_architecture, resolve
    from jax_vllm_amd.parts import DecoderModel, LayerRun, LayerSpec, ModelSpec, PartSpec, register_part
    from jax_vllm_amd.weights.loader import TORCH_DTYPES, target_dtype

    register_part("mixer", "running_mean", RunningMeanMixer)
    register_part("mixer", "running_mean_on_device", RunningMeanMixerOnDevice)
    hidden, vocab, inter = TOY_STATE["hidden"], TOY_STATE["vocab"], TOY_STATE["inter"]
    norm = PartSpec("rmsnorm", {"size": hidden, "eps": 1e-5})
    att = PartSpec("gqa_attention", dict(hidden_size=hidden, num_heads=3, num_kv_heads=1, head_dim=16, qk_norm_eps=1e-5,
                                         position=PartSpec("rotary", {"head_dim": 16, "theta": 1e4})))
    toy = PartSpec(mixer_kind, {"hidden_size": hidden})
    ffn = PartSpec("gated_mlp", {"hidden_size": hidden, "intermediate_size": inter})

    def build(_cfg):
        return ModelSpec(
            vocab_size=vocab, hidden_size=hidden,
            embedding=PartSpec("token_embedding", {"vocab_size": vocab, "hidden_size": hidden}), embedding_prefix="emb.",
            final_norm=norm, final_norm_prefix="norm.", head=PartSpec("linear_head", {"vocab_size": vocab, "hidden_size": hidden}),
            head_prefix="head.", tie_head_to_embedding=True,
            layers=[LayerSpec(f"l{i}.", mixer, ffn, PartSpec("prenorm", {"norm": norm}), "mix.", "ffn.")
                    for i, mixer in enumerate([toy, att, toy])],
            schedule=[LayerRun(0), LayerRun(1), LayerRun(2), LayerRun(0)])

    register_architecture("ToyStateModel", lambda c: c, build)
    arch, cfg, _ = resolve({"architectures": ["ToyStateModel"]})
    model = DecoderModel(arch.build_spec(cfg))
    g = torch.Generator().manual_seed(13)
    compute = TORCH_DTYPES[dtype]
    w = {n: ((0.2 * torch.randn(ts.shape, generator=g)) if ts.role == "matrix" else 1 + 0.1 * torch.randn(ts.shape, generator=g))
         .to(torch.bfloat16).float() for n, ts in model.tensor_specs().items()}
    model.bind({n: v.cuda().to(target_dtype(model.tensor_specs()[n].role, compute)) for n, v in w.items()}, compute)
    return model, w


TOY_STATE = dict(hidden=48, vocab=120, inter=96)


def toy_state_plain(w, tokens):
    """The toy model written out whole: no state, a cumulative mean over the sequence."""
    t = len(tokens)
    pos = torch.arange(t)
    c = dict(num_heads=3, num_kv_heads=1, head_dim=16, rms_norm_eps=1e-5, rope_theta=1e4)
    h = w["emb.weight"][torch.tensor(tokens)]
    for i in (0, 1, 2, 0):
        x = P.rms_norm(w[f"l{i}.input_layernorm.weight"], 1e-5, h)
        if i == 1:
            a = P.attention_block(w, "l1.mix", c, x, pos)
        else:
            a = (torch.cumsum(x, 0) / torch.arange(1, t + 1)[:, None]) @ w[f"l{i}.mix.proj.weight"].T
        h = h + a
        m = P.rms_norm(w[f"l{i}.post_attention_layernorm.weight"], 1e-5, h)
        h = h + P.swiglu(w[f"l{i}.ffn.gate_proj.weight"], w[f"l{i}.ffn.up_proj.weight"], w[f"l{i}.ffn.down_proj.weight"], m)
    return (P.rms_norm(w["norm.weight"], 1e-5, h) @ w["emb.weight"].T).numpy()


@pytest.mark.parametrize("graphs", [False, True], ids=["eager", "graphs-on"])
@pytest.mark.parametrize("dtype", DTYPES)
def test_toy_mixer_with_state_is_registered_built_and_stepped(folders, dtype, graphs):
    """With HIP graphs switched on as well: the mixer plans on the host and has not declared
    itself replayable, so every step runs eagerly with its true slots."""
    hidden, vocab = TOY_STATE["hidden"], TOY_STATE["vocab"]
    model, w = toy_state_model(dtype, "running_mean")
    core = make_core(None, dtype, 8, pages=24, seqs=3, model=model, graphs=graphs)
    assert [p.state is not None for p in core.plan] == [True, False, True, True]
    assert not core.cache.prefix_cache                      # state forbids taking pages over
    assert not model.replayable()
    # one row per slot and the spare row
    assert [m.state.shape for m in core.memories if m.state is not None] == [(4, hidden)] * 3

    def plain(tokens):
        return toy_state_plain(w, tokens)

    rng = np.random.default_rng(6)
    reqs = {r: rng.integers(0, vocab, size=n).tolist() for r, n in (("a", 40), ("b", 23), ("c", 31))}
    fed = {r: 0 for r in reqs}
    got = {r: [] for r in reqs}
    for r in reqs:
        core.start_request(r)
    cuts = [[("a", 7)], [("a", 2), ("b", 9)], [("b", 1), ("c", 31), ("a", 1)], [("a", 20), ("b", 8)]]
    cuts += [[("a", 1), ("b", 1)]] * 5 + [[("a", 1)]] * 5       # the tails one by one: steps a graph engine would record
    for step in cuts:
        es = [entry(r, reqs[r][fed[r]:fed[r] + n]) for r, n in step]
        out = core.run(es).cpu().numpy()
        at = 0
        for r, n in step:
            got[r].append(out[at:at + n])
            at += n
            fed[r] += n
    assert core.graph_replays == 0 and not core._graphs
    for r in reqs:
        assert fed[r] == len(reqs[r])
        check_logits(dtype, np.concatenate(got[r]), plain(reqs[r]), what=r)
    # a slot that is given back and taken again starts from zero state
    core.finish_request("b")
    core.start_request("d")
    out = core.run([entry("d", reqs["c"])]).cpu().numpy()
    check_logits(dtype, out, plain(reqs["c"]), what="d after b")


@pytest.mark.parametrize("dtype", DTYPES)
def test_toy_mixer_with_state_on_the_device_is_recorded_and_replayed(dtype):
    """The same toy model with a mixer that declares ``replayable``: its decode steps are recorded
    and replayed.  Three live requests make a step of four rows: the padding row writes the spare
    state row, never a request's; requests end and their slots are taken again from zero."""
    vocab = TOY_STATE["vocab"]
    model, w = toy_state_model(dtype, "running_mean_on_device")
    assert model.replayable()
    core = make_core(None, dtype, 8, pages=40, seqs=4, model=model, graphs=True)
    rng = np.random.default_rng(7)
    reqs = {r: rng.integers(0, vocab, size=n).tolist() for r, n in (("a", 40), ("b", 33), ("c", 36), ("d", 30), ("e", 25))}
    want = {r: toy_state_plain(w, t) for r, t in reqs.items()}
    fed, got = {}, {r: [] for r in reqs}

    def admit(r, n):
        core.start_request(r)
        got[r].append(core.run([entry(r, reqs[r][:n])]).cpu().numpy())
        fed[r] = n

    def decode():
        live = [r for r in fed if fed[r] < len(reqs[r])]
        out = core.run([entry(r, reqs[r][fed[r]:fed[r] + 1]) for r in live]).cpu().numpy()
        for i, r in enumerate(live):
            got[r].append(out[i:i + 1])
            fed[r] += 1
            if fed[r] == len(reqs[r]):
                core.finish_request(r)
        return len(live)

    admit("a", 9), admit("b", 17), admit("c", 5)
    for _ in range(16):
        assert decode() == 3                    # four rows, one of them padding
    admit("d", 11)                               # slot 3
    while fed["b"] < len(reqs["b"]):
        decode()
    admit("e", 8)                                # b's slot again: zeroed
    while any(fed[r] < len(reqs[r]) for r in fed):
        decode()
    assert core.graph_replays >= 30
    for r in reqs:
        check_logits(dtype, np.concatenate(got[r]), want[r], what=r)
    spare = [m.state[-1] for m in core.memories if m.state is not None]
    assert any(float(s.abs().max()) > 0 for s in spare)      # the padding rows did write there


class TopOneExperts:
    """A toy feed-forward with routing, defined and registered here: router logits in float, the
    best expert of each token (lowest index on ties) runs a two-matrix ReLU feed-forward and its
    output is scaled by the router's softmax weight of that expert."""

    def __init__(self, hidden_size: int, intermediate_size: int, num_experts: int):
        self.h, self.i, self.e = hidden_size, intermediate_size, num_experts

    def tensors(self):
        from jax_vllm_amd.parts import TensorSpec

        t = {"router.weight": TensorSpec((self.e, self.h))}
        for x in range(self.e):
            t[f"experts.{x}.up.weight"] = TensorSpec((self.i, self.h))
            t[f"experts.{x}.down.weight"] = TensorSpec((self.h, self.i))
        return t

    def bind(self, tensors, dtype):
        self.t = tensors

    def forward(self, x, ctx):
        logits = x.float() @ self.t["router.weight"].float().t()
        weight, choice = torch.softmax(logits, dim=-1).max(dim=-1)
        out = torch.zeros_like(x)
        for e in range(self.e):
            rows = (choice == e).nonzero().flatten()
            if rows.numel():
                hid = torch.relu(x[rows] @ self.t[f"experts.{e}.up.weight"].t())
                out[rows] = ((hid @ self.t[f"experts.{e}.down.weight"].t()).float() * weight[rows, None]).to(x.dtype)
        return out


class LinearFrequencyRotation:
    """A toy position encoding, defined and registered here: neighbouring pairs (2i, 2i+1) of the
    first ``rotary_dim`` head elements turn by position * (i + 1) * step; the rest pass through."""

    def __init__(self, rotary_dim: int, step: float):
        self.rotary_dim, self.step = rotary_dim, step

    def tensors(self):
        return {}

    def bind(self, tensors, dtype, device=None):
        self.freq = (torch.arange(1, self.rotary_dim // 2 + 1, dtype=torch.float32) * self.step).to(device or "cuda")

    def as_rotation(self):
        return self.rotary_dim, True

    def rotation_table(self, ctx):
        from jax_vllm_amd.ops import kernels as K

        key = ("linear_frequency_table", self.rotary_dim, self.step)
        if key not in ctx.extras:
            ctx.extras[key] = K.rope_table(ctx.positions, self.freq)
        return ctx.extras[key]


@pytest.mark.parametrize("dtype", DTYPES)
def test_toy_routed_feed_forward_and_toy_position_encoding(dtype):
    """Layers pick their parts one by one: a routed feed-forward in one layer, a dense one in the
    other, and attention with a position encoding of the test's own, all without a change to the
    package.  The plain implementation is written out here."""
    from jax_vllm_amd.config import register_architecture, resolve
    from jax_vllm_amd.parts import DecoderModel, LayerRun, LayerSpec, ModelSpec, PartSpec, register_part
    from jax_vllm_amd.weights.loader import TORCH_DTYPES, target_dtype

    register_part("feed_forward", "top_one_experts", TopOneExperts)
    register_part("position", "linear_frequency", LinearFrequencyRotation)
    hidden, vocab, inter, heads, kvh, d, rot, step, eps = 40, 90, 56, 4, 2, 16, 8, 0.37, 1e-5
    norm = PartSpec("rmsnorm", {"size": hidden, "eps": eps})
    att = PartSpec("gqa_attention", dict(hidden_size=hidden, num_heads=heads, num_kv_heads=kvh, head_dim=d, qk_norm_eps=eps,
                                         position=PartSpec("linear_frequency", {"rotary_dim": rot, "step": step})))
    routed = PartSpec("top_one_experts", {"hidden_size": hidden, "intermediate_size": inter, "num_experts": 3})
    dense = PartSpec("gated_mlp", {"hidden_size": hidden, "intermediate_size": inter})

    def build(_cfg):
        return ModelSpec(
            vocab_size=vocab, hidden_size=hidden,
            embedding=PartSpec("token_embedding", {"vocab_size": vocab, "hidden_size": hidden}), embedding_prefix="emb.",
            final_norm=norm, final_norm_prefix="norm.", head=PartSpec("linear_head", {"vocab_size": vocab, "hidden_size": hidden}),
            head_prefix="head.", tie_head_to_embedding=False,
            layers=[LayerSpec(f"l{i}.", att, ff, PartSpec("prenorm", {"norm": norm}), "att.", "ff.")
                    for i, ff in enumerate([routed, dense])],
            schedule=[LayerRun(0), LayerRun(1)])

    register_architecture("ToyRoutedModel", lambda c: c, build)
    arch, cfg, _ = resolve({"architectures": ["ToyRoutedModel"]})
    model = DecoderModel(arch.build_spec(cfg))
    g = torch.Generator().manual_seed(21)
    compute = TORCH_DTYPES[dtype]
    w = {n: ((0.25 * torch.randn(ts.shape, generator=g)) if ts.role == "matrix" else 1 + 0.1 * torch.randn(ts.shape, generator=g))
         .to(torch.bfloat16).float() for n, ts in model.tensor_specs().items()}
    # the router separates its experts clearly, so that rounding does not flip a choice
    w["l0.ff.router.weight"] = (w["l0.ff.router.weight"] * 6).to(torch.bfloat16).float()
    model.bind({n: v.cuda().to(target_dtype(model.tensor_specs()[n].role, compute)) for n, v in w.items()}, compute)
    core = make_core(None, dtype, 8, pages=30, seqs=2, model=model)

    def rotate(x, pos):                      # x [heads, T, d]
        ang = pos[:, None].float() * (torch.arange(1, rot // 2 + 1).float() * step)[None, :]
        cos, sin = torch.cos(ang)[None], torch.sin(ang)[None]
        a, b = x[..., 0:rot:2], x[..., 1:rot:2]
        y = x.clone()
        y[..., 0:rot:2] = a * cos - b * sin
        y[..., 1:rot:2] = b * cos + a * sin
        return y

    def attention(p, x, pos):
        t = x.shape[0]
        q = (x @ w[f"{p}.q_proj.weight"].T).reshape(t, heads, d).transpose(0, 1)
        k = (x @ w[f"{p}.k_proj.weight"].T).reshape(t, kvh, d).transpose(0, 1)
        v = (x @ w[f"{p}.v_proj.weight"].T).reshape(t, kvh, d).transpose(0, 1)
        q = rotate(P.rms_norm(w[f"{p}.q_norm.weight"], eps, q), pos)
        k = rotate(P.rms_norm(w[f"{p}.k_norm.weight"], eps, k), pos)
        o = P.attention_core(q, k, v, P.causal_mask(t, t)).transpose(0, 1).reshape(t, heads * d)
        return o @ w[f"{p}.o_proj.weight"].T

    def experts(p, x):
        probs = torch.softmax(x @ w[f"{p}.router.weight"].T, dim=-1)
        weight, choice = probs.max(dim=-1)
        out = torch.zeros_like(x)
        for t in range(x.shape[0]):
            e = int(choice[t])
            out[t] = (torch.relu(x[t] @ w[f"{p}.experts.{e}.up.weight"].T) @ w[f"{p}.experts.{e}.down.weight"].T) * weight[t]
        return out, choice

    def plain(tokens):
        pos = torch.arange(len(tokens))
        h = w["emb.weight"][torch.tensor(tokens)]
        choices = None
        for i in (0, 1):
            h = h + attention(f"l{i}.att", P.rms_norm(w[f"l{i}.input_layernorm.weight"], eps, h), pos)
            m = P.rms_norm(w[f"l{i}.post_attention_layernorm.weight"], eps, h)
            if i == 0:
                delta, choices = experts("l0.ff", m)
            else:
                delta = P.swiglu(w["l1.ff.gate_proj.weight"], w["l1.ff.up_proj.weight"], w["l1.ff.down_proj.weight"], m)
            h = h + delta
        return (P.rms_norm(w["norm.weight"], eps, h) @ w["head.weight"].T).numpy(), choices

    rng = np.random.default_rng(8)
    toks = rng.integers(0, vocab, size=70).tolist()
    want, choices = plain(toks)
    assert len(set(choices.tolist())) == 3                   # every expert is used
    # a shift of all positions changes nothing where only distances count: the oracle's own check
    # of its rotation (a wrong pairing or sign fails it)
    x = torch.randn(heads, 5, d, generator=g)
    s0 = torch.einsum("hqd,hkd->hqk", rotate(x, torch.arange(5)), rotate(x, torch.arange(5)))
    s9 = torch.einsum("hqd,hkd->hqk", rotate(x, torch.arange(9, 14)), rotate(x, torch.arange(9, 14)))
    torch.testing.assert_close(s0, s9, rtol=1e-4, atol=1e-4)
    core.start_request("a")
    got, at = [], 0
    for n in [19, 2, 1, 30, 1, 1, 16]:
        got.append(core.run([entry("a", toks[at:at + n])]).cpu().numpy())
        at += n
    assert at == len(toks)
    check_logits(dtype, np.concatenate(got), want)


# ------------------------------------------------------------------ an embedding that reads the step's positions; a mixer with a cache of its own shape
class PositionedEmbedding:
    """A toy embedding, defined and registered here: token row plus a learned row per absolute
    position.  It takes the positions from the step's context on the device, so it may be replayed."""

    replayable = True

    def __init__(self, vocab_size: int, hidden_size: int, max_positions: int):
        self.v, self.h, self.n = vocab_size, hidden_size, max_positions

    def tensors(self):
        from jax_vllm_amd.parts import TensorSpec

        return {"weight": TensorSpec((self.v, self.h)), "positions.weight": TensorSpec((self.n, self.h))}

    def bind(self, tensors, dtype):
        self.weight, self.rows = tensors["weight"], tensors["positions.weight"]

    def forward(self, ids, ctx):
        return self.weight[ids.long()].float() + self.rows[ctx.positions.long()].float()


class LatentMeanMixer:
    """A toy mixer with a paged cache that is no key/value pair: per token it stores ONE latent
    vector of ``latent`` floats (always float32, token-major pages), and its output at a token is a
    projection of the mean of the latents of all tokens up to it, read back from the pages through
    the block table.  Plans on the host; never replayed."""

    def __init__(self, hidden_size: int, latent: int):
        self.h, self.r = hidden_size, latent

    def tensors(self):
        from jax_vllm_amd.parts import TensorSpec

        return {"down.weight": TensorSpec((self.r, self.h)), "up.weight": TensorSpec((self.h, self.r))}

    def cache_spec(self):
        from jax_vllm_amd.parts import PagedCacheSpec, PagedTensorSpec

        return PagedCacheSpec((PagedTensorSpec("latent", (self.r,), slot_axis=0, dtype="float32"),))

    def state_spec(self):
        return None

    def bind(self, tensors, dtype):
        self.down, self.up = tensors["down.weight"], tensors["up.weight"]

    def forward(self, x, ctx, mem):
        store = mem.pages["latent"]                       # [pages + 1, page_size, latent]
        flat = store.view(-1, self.r)
        if mem.writes:                                    # a run that reads another run's cache stores nothing
            flat[ctx.slot_mappings[mem.group].long()] = (x @ self.down.t()).float()
        out = torch.empty_like(x)
        tables = ctx.block_tables[mem.group]
        at = 0
        for i, (q, c) in enumerate(zip(ctx.q_lens_host, ctx.context_lens_host)):
            seen = store[tables[i].long()].reshape(-1, self.r)[:c + q]        # the request's latents in order
            means = torch.cumsum(seen, 0)[c:] / torch.arange(c + 1, c + q + 1, device=x.device)[:, None]
            out[at:at + q] = (means.to(x.dtype) @ self.up.t()).to(x.dtype)
            at += q
        return out


def _bound_toy(name, spec_builder, dtype, seed, scale=0.2):
    from jax_vllm_amd.config import register_architecture, resolve
    from jax_vllm_amd.parts import DecoderModel
    from jax_vllm_amd.weights.loader import TORCH_DTYPES, target_dtype

    register_architecture(name, lambda c: c, spec_builder)
    arch, cfg, _ = resolve({"architectures": [name]})
    model = DecoderModel(arch.build_spec(cfg))
    g = torch.Generator().manual_seed(seed)
    compute = TORCH_DTYPES[dtype]
    w = {n: ((scale * torch.randn(ts.shape, generator=g)) if ts.role == "matrix" else 1 + 0.1 * torch.randn(ts.shape, generator=g))
         .to(torch.bfloat16).float() for n, ts in model.tensor_specs().items()}
    model.bind({n: v.cuda().to(target_dtype(model.tensor_specs()[n].role, compute)) for n, v in w.items()}, compute)
    return model, w


@pytest.mark.parametrize("graphs", [False, True], ids=["eager", "graphs-on"])
@pytest.mark.parametrize("dtype", DTYPES)
def test_toy_embedding_with_learned_positions_and_attention_without_rotation(dtype, graphs):
    """The embedding part gets the step's context: a learned row per absolute position is added
    there, and the attention runs with no position part at all.  Nothing of the package changes."""
    from jax_vllm_amd.parts import LayerRun, LayerSpec, ModelSpec, PartSpec, register_part

    register_part("embedding", "positioned_embedding", PositionedEmbedding)
    hidden, vocab, inter, heads, kvh, d, eps, npos = 56, 75, 72, 4, 2, 16, 1e-5, 128
    norm = PartSpec("rmsnorm", {"size": hidden, "eps": eps})
    att = PartSpec("gqa_attention", dict(hidden_size=hidden, num_heads=heads, num_kv_heads=kvh, head_dim=d, qk_norm_eps=eps))

    def build(_cfg):
        return ModelSpec(
            vocab_size=vocab, hidden_size=hidden,
            embedding=PartSpec("positioned_embedding", {"vocab_size": vocab, "hidden_size": hidden, "max_positions": npos}),
            embedding_prefix="emb.", final_norm=norm, final_norm_prefix="norm.",
            head=PartSpec("linear_head", {"vocab_size": vocab, "hidden_size": hidden}), head_prefix="head.",
            layers=[LayerSpec(f"l{i}.", att, PartSpec("gated_mlp", {"hidden_size": hidden, "intermediate_size": inter}),
                              PartSpec("prenorm", {"norm": norm}), "att.", "ff.") for i in range(2)],
            schedule=[LayerRun(0), LayerRun(1)])

    model, w = _bound_toy("ToyPositionedModel", build, dtype, 31)
    assert model.replayable()

    def plain(tokens):
        t = len(tokens)
        h = w["emb.weight"][torch.tensor(tokens)] + w["emb.positions.weight"][:t]
        for i in (0, 1):
            p = f"l{i}.att"
            x = P.rms_norm(w[f"l{i}.input_layernorm.weight"], eps, h)
            q = P.rms_norm(w[f"{p}.q_norm.weight"], eps, (x @ w[f"{p}.q_proj.weight"].T).reshape(t, heads, d).transpose(0, 1))
            k = P.rms_norm(w[f"{p}.k_norm.weight"], eps, (x @ w[f"{p}.k_proj.weight"].T).reshape(t, kvh, d).transpose(0, 1))
            v = (x @ w[f"{p}.v_proj.weight"].T).reshape(t, kvh, d).transpose(0, 1)
            o = P.attention_core(q, k, v, P.causal_mask(t, t)).transpose(0, 1).reshape(t, heads * d)
            h = h + o @ w[f"{p}.o_proj.weight"].T
            m = P.rms_norm(w[f"l{i}.post_attention_layernorm.weight"], eps, h)
            h = h + P.swiglu(w[f"l{i}.ff.gate_proj.weight"], w[f"l{i}.ff.up_proj.weight"], w[f"l{i}.ff.down_proj.weight"], m)
        return (P.rms_norm(w["norm.weight"], eps, h) @ w["head.weight"].T).numpy()

    core = make_core(None, dtype, 8, pages=30, seqs=3, model=model, graphs=graphs)
    rng = np.random.default_rng(9)
    reqs = {r: rng.integers(0, vocab, size=n).tolist() for r, n in (("a", 60), ("b", 41))}
    # without its position rows the model would not tell a sequence from a permutation of it: the
    # oracle's answer must depend on them
    assert np.abs(plain(reqs["b"])[-1] - plain(reqs["b"][::-1][:-1] + reqs["b"][-1:])[-1]).max() > 1e-3
    fed, got = {r: 0 for r in reqs}, {r: [] for r in reqs}
    for r in reqs:
        core.start_request(r)
    cuts = [[("a", 9)], [("a", 30), ("b", 22)], [("a", 1), ("b", 2)]] + [[("a", 1), ("b", 1)]] * 17 + [[("a", 1)]] * 3
    for step in cuts:
        out = core.run([entry(r, reqs[r][fed[r]:fed[r] + n]) for r, n in step]).cpu().numpy()
        at = 0
        for r, n in step:
            got[r].append(out[at:at + n])
            at, fed[r] = at + n, fed[r] + n
    assert (core.graph_replays > 10) == graphs
    for r in reqs:
        assert fed[r] == len(reqs[r])
        check_logits(dtype, np.concatenate(got[r]), plain(reqs[r]), what=r)


@pytest.mark.parametrize("dtype", DTYPES)
def test_toy_mixer_declares_a_paged_cache_of_its_own_shape(dtype):
    """A mixer says what it keeps per token; the storage gives it exactly that (one float32 tensor,
    token-major pages), in a page group that it shares with an attention layer (same need: all
    earlier tokens), and pages are taken again after requests end."""
    from jax_vllm_amd.parts import LayerRun, LayerSpec, ModelSpec, PartSpec, register_part

    register_part("mixer", "latent_mean", LatentMeanMixer)
    hidden, vocab, inter, latent, eps, ps = 48, 66, 64, 12, 1e-5, 8
    norm = PartSpec("rmsnorm", {"size": hidden, "eps": eps})
    att = PartSpec("gqa_attention", dict(hidden_size=hidden, num_heads=3, num_kv_heads=1, head_dim=16, qk_norm_eps=eps,
                                         position=PartSpec("rotary", {"head_dim": 16, "theta": 1e4})))
    toy = PartSpec("latent_mean", {"hidden_size": hidden, "latent": latent})
    ffn = PartSpec("gated_mlp", {"hidden_size": hidden, "intermediate_size": inter})

    def build(_cfg):
        return ModelSpec(
            vocab_size=vocab, hidden_size=hidden,
            embedding=PartSpec("token_embedding", {"vocab_size": vocab, "hidden_size": hidden}), embedding_prefix="emb.",
            final_norm=norm, final_norm_prefix="norm.", head=PartSpec("linear_head", {"vocab_size": vocab, "hidden_size": hidden}),
            head_prefix="head.", tie_head_to_embedding=True,
            layers=[LayerSpec(f"l{i}.", mixer, ffn, PartSpec("prenorm", {"norm": norm}), "mix.", "ffn.")
                    for i, mixer in enumerate([toy, att])],
            schedule=[LayerRun(0), LayerRun(1), LayerRun(0, cache_of=0)])    # the third run reads the first run's latents

    model, w = _bound_toy("ToyLatentModel", build, dtype, 37)
    core = make_core(None, dtype, ps, pages=12, seqs=3, model=model)
    assert core.group_keys == [("full",)]
    toy_mem, att_mem, reader = core.memories
    assert list(toy_mem.pages) == ["latent"] and toy_mem.pages["latent"].shape == (13, ps, latent)
    assert toy_mem.pages["latent"].dtype == torch.float32
    assert sorted(att_mem.pages) == ["k", "v"] and att_mem.pages["k"].dtype == core.dtype
    assert reader.pages is toy_mem.pages and not reader.writes
    item = 4 if dtype == "float32" else 2
    assert core.kv_bytes_per_token == latent * 4 + 2 * 16 * item

    def plain(tokens):
        t = len(tokens)
        c = dict(num_heads=3, num_kv_heads=1, head_dim=16, rms_norm_eps=eps, rope_theta=1e4)
        h = w["emb.weight"][torch.tensor(tokens)]
        first = None
        for run, i in enumerate((0, 1, 0)):
            x = P.rms_norm(w[f"l{i}.input_layernorm.weight"], eps, h)
            if i == 1:
                a = P.attention_block(w, "l1.mix", c, x, torch.arange(t))
            else:
                lat = x @ w["l0.mix.down.weight"].T
                first = lat if first is None else first          # the reader run mixes the owner's latents
                a = (torch.cumsum(first, 0) / torch.arange(1, t + 1)[:, None]) @ w["l0.mix.up.weight"].T
            h = h + a
            m = P.rms_norm(w[f"l{i}.post_attention_layernorm.weight"], eps, h)
            h = h + P.swiglu(w[f"l{i}.ffn.gate_proj.weight"], w[f"l{i}.ffn.up_proj.weight"], w[f"l{i}.ffn.down_proj.weight"], m)
        return (P.rms_norm(w["norm.weight"], eps, h) @ w["emb.weight"].T).numpy()

    rng = np.random.default_rng(10)
    reqs = {r: rng.integers(0, vocab, size=n).tolist() for r, n in (("a", 37), ("b", 30), ("c", 44), ("d", 25))}
    fed, got = {r: 0 for r in reqs}, {r: [] for r in reqs}
    cuts = [[("a", 11)], [("a", 2), ("b", 17)], [("a", 24), ("b", 1)], [("b", 12)],       # a and b end: 9 of 12 pages go back
            [("c", 30)], [("c", 1), ("d", 9)], [("c", 13), ("d", 16)]]
    for step in cuts:
        for r, _ in step:
            if not core.has_request(r):
                core.start_request(r)
        out = core.run([entry(r, reqs[r][fed[r]:fed[r] + n]) for r, n in step]).cpu().numpy()
        at = 0
        for r, n in step:
            got[r].append(out[at:at + n])
            at, fed[r] = at + n, fed[r] + n
            if fed[r] == len(reqs[r]):
                core.finish_request(r)
        core.cache.check_invariants()
    assert core.cache.num_free_pages(0) == 12
    for r in reqs:
        assert fed[r] == len(reqs[r])
        check_logits(dtype, np.concatenate(got[r]), plain(reqs[r]), what=r)


# ------------------------------------------------------------------ steps started ahead with a window group, and with state
def _tokens_follow(dtype, plain_logits, prompt, tokens, what=""):
    """Every token is the plain implementation's choice given all before it (one whole-sequence pass:
    the models are causal); in bfloat16 a token within 4 % of the maximum is accepted."""
    logits = plain_logits(list(prompt) + list(tokens[:-1]))[len(prompt) - 1:]
    for k, t in enumerate(tokens):
        margin = float(logits[k].max() - logits[k][t])
        allowed = (1e-5 if dtype == "float32" else 0.04) * float(np.abs(logits[k]).max())
        assert margin <= allowed, f"{what} token {k}: engine's {t} is {margin} below the plain maximum"


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("kind", ["window", "state"])
def test_decode_steps_started_ahead_with_a_window_group_and_with_state(folders, dtype, kind):
    """Steps started ahead of their tokens on models whose cache changes between such steps: a window
    group gives pages back when a token is committed (the table rows of the recorded step move
    while the next step is already under way), a mixer with state on the device keeps a row per slot
    and the padding rows write the spare one.  Requests end on an eos_id while a step is under way
    and their slots are taken again.  Tokens equal those of an engine that waits for every step,
    and follow the plain implementation."""
    from jax_vllm_amd import LLM, SamplingParams

    if kind == "window":
        cfg, w = plain_of(folders["B"])
        schedule, windows = [(0, None), (1, None), (2, None)], {1: 20}
        model = custom_model(folders["B"], dtype, schedule, windows)
        vocab = cfg["vocab_size"]

        def plain(seq):
            return P.forward_scheduled(w, cfg, seq, schedule, windows).numpy()
    else:
        model, w = toy_state_model(dtype, "running_mean_on_device")
        vocab = TOY_STATE["vocab"]

        def plain(seq):
            return toy_state_plain(w, seq)
    rng = np.random.default_rng(23)
    prompts = [rng.integers(0, vocab, size=n).tolist() for n in (30, 7, 12, 9, 21)]
    # what the third request would say first: one of its early tokens ends it, in the middle of followed steps
    probe = LLM(model, dtype=dtype, block_size=8, max_num_seqs=3, max_model_len=128, max_num_batched_tokens=64,
                decode_ahead=False)
    eos = probe.generate([prompts[2]], SamplingParams(max_new_tokens=12))[0][9]
    params = [SamplingParams(max_new_tokens=70), SamplingParams(max_new_tokens=64), SamplingParams(max_new_tokens=40, eos_id=eos),
              SamplingParams(max_new_tokens=30), SamplingParams(max_new_tokens=25)]
    outs = {}
    for ahead in (False, True):
        llm = LLM(model, dtype=dtype, block_size=8, max_num_seqs=3, max_model_len=128, max_num_batched_tokens=64,
                  decode_ahead=ahead)
        assert llm.core._replayable
        outs[ahead] = llm.generate(prompts, params)          # five requests over three slots: slots are taken again
        assert (llm.core.steps_followed > 30) == ahead and llm.core.graph_replays > 30
        llm.core.cache.check_invariants()
        assert not llm.core.cache.requests
        for g in range(len(llm.core.group_keys)):
            assert llm.core.cache.num_free_pages(g) == llm.config.usable_pages
    # a request that waits for the slot of one that ends on its eos_id is admitted one step later when steps
    # are started ahead, so the steps hold other rows: in float32 that changes no token, in bfloat16 the
    # rounding of other kernel choices may turn a near-tie, and each engine is held to the plain tokens instead
    if dtype == "float32":
        assert outs[True] == outs[False]
    for ahead in (False, True):
        assert len(outs[ahead][2]) <= 10 and outs[ahead][2][-1] == eos
        assert [len(o) for i, o in enumerate(outs[ahead]) if i != 2] == [70, 64, 30, 25]
        for i, (p, o) in enumerate(zip(prompts, outs[ahead])):
            _tokens_follow(dtype, plain, p, o, what=f"request {i} (ahead={ahead})")


def test_prewarm_with_the_library_timing_its_own_kernels(folders):
    """``tune_library``: during ``prewarm`` (and only then) the matrix library times its own kernels for the
    products it is given.  Afterwards its timing pass is off again, and the tokens are the plain ones."""
    from jax_vllm_amd import LLM, SamplingParams

    cfg, w = plain_of(folders["B"])
    rng = np.random.default_rng(31)
    prompts = [rng.integers(0, cfg["vocab_size"], size=n).tolist() for n in (40, 23, 31)]
    was = (torch.cuda.tunable.is_enabled(), torch.cuda.tunable.tuning_is_enabled())
    try:
        llm = LLM(folders["B"], dtype="bfloat16", block_size=16, max_num_seqs=24, max_model_len=128,
                  max_num_batched_tokens=64, tune_library=True)
        assert llm.prewarm() > 0
        assert torch.cuda.tunable.is_enabled() and not torch.cuda.tunable.tuning_is_enabled()
        got = llm.generate(prompts, SamplingParams(max_new_tokens=12))
        for p, g in zip(prompts, got):
            check_tokens_follow("bfloat16", cfg, w, p, g)
    finally:
        torch.cuda.tunable.tuning_enable(was[1])
        torch.cuda.tunable.enable(was[0])
