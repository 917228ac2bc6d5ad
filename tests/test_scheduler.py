"""The scheduler's decisions, on the host alone: the real cache manager and the real loop,
with a stand-in for the step function whose "model" is a fixed function of a request's whole
token sequence, so that the expected output does not depend on how the work was cut."""
import hashlib

import numpy as np
import pytest

from jax_vllm_amd.cache import CacheManager
from jax_vllm_amd.config import EngineConfig
from jax_vllm_amd.engine.llm import Engine
from jax_vllm_amd.engine.request import SamplingParams

VOCAB = 97


def next_token(seq) -> int:
    return int.from_bytes(hashlib.sha256(repr(list(seq)).encode()).digest()[:4], "little") % VOCAB


def expected(prompt, n, eos=None):
    seq, out = list(prompt), []
    for _ in range(n):
        t = next_token(seq)
        out.append(t)
        seq.append(t)
        if eos is not None and t == eos:
            break
    return out


class FakeCore:
    """Does to the cache manager what the step function does, and logs every step."""

    def __init__(self, cfg, groups=(("full",),)):
        self.cache = CacheManager(list(groups), cfg.page_size, cfg.usable_pages, cfg.max_num_seqs,
                                  cfg.enable_prefix_cache)
        self.steps = []

    def run(self, entries, borrow=False):
        for e in entries:
            self.cache.reserve(e.request_id, len(e.tokens))
        rows, log = [], []
        for e in entries:
            ctx = self.cache.requests[e.request_id].tokens
            log.append((e.request_id, len(ctx), len(e.tokens), list(e.want)))
            rows += [next_token(ctx + list(e.tokens[:w + 1])) for w in e.want]
        for e in entries:
            self.cache.commit(e.request_id, e.tokens)
        self.cache.check_invariants()
        self.steps.append(log)
        return rows

    @staticmethod
    def sample(rows, temps, keys):
        assert len(rows) == len(temps) == len(keys)
        return rows


def make(**kw):
    cfg = EngineConfig(**kw)
    core = FakeCore(cfg)
    return Engine(cfg, core.cache, core.run, core.sample, VOCAB), core


def drain(eng, limit=5000):
    events = []
    while eng.has_work():
        events.append(eng.step())
        limit -= 1
        assert limit > 0, "the engine does not finish"
    return events


def test_two_requests_share_one_step_and_budget_is_respected():
    eng, core = make(block_size=4, max_num_seqs=4, max_model_len=64, max_num_batched_tokens=16)
    a = eng.add_request(list(range(10)), SamplingParams(max_new_tokens=3))
    b = eng.add_request(list(range(20, 29)), SamplingParams(max_new_tokens=3))
    drain(eng)
    # step 0: a whole (10 tokens) and the first 6 of b under the budget of 16; step 1: a decodes
    # first (one token), then b's remaining 3 tokens
    assert core.steps[0] == [(a, 0, 10, [9]), (b, 0, 6, [])]
    assert core.steps[1] == [(a, 10, 1, [0]), (b, 6, 3, [2])]
    assert all(sum(n for _, _, n, _ in s) <= 16 for s in core.steps)
    assert eng.stats.max_batched_tokens == 16 and eng.stats.admissions == 2
    assert eng.stats.emitted_tokens == 6 and eng.stats.decode_tokens == 4 and eng.stats.prefill_tokens == 19


def test_outputs_do_not_depend_on_budget_chunk_or_pages():
    rng = np.random.default_rng(0)
    prompts = [rng.integers(0, VOCAB, size=n).tolist() for n in (1, 9, 40, 64, 100)]
    want = [expected(p, 12) for p in prompts]
    for kw in (dict(max_num_batched_tokens=2048), dict(max_num_batched_tokens=24), dict(max_num_batched_tokens=7, max_chunk=3),
               dict(max_num_batched_tokens=24, num_blocks=1 + 12), dict(max_num_batched_tokens=5, num_blocks=1 + 8, max_num_seqs=2)):
        eng, core = make(**dict(dict(block_size=16, max_num_seqs=4, max_model_len=128), **kw))
        got = eng.generate(prompts, SamplingParams(max_new_tokens=12))
        assert got == want, kw
        assert core.cache.num_free_pages() == eng.config.usable_pages and core.cache.slots.num_free == eng.config.max_num_seqs


def test_chunk_count_and_first_token_step():
    """ceil(T / chunk) portions; the first token comes from the step that ends the prompt
    (reference: jllm/engine/engine.py:391-403, tests/test_engine.py:129-186)."""
    eng, core = make(block_size=16, max_num_seqs=1, max_model_len=128, max_num_batched_tokens=16)
    eng.add_request(list(range(50)), SamplingParams(max_new_tokens=2))
    events = drain(eng)
    assert [len(e) for e in events] == [0, 0, 0, 1, 1]
    assert [s[0][2] for s in core.steps] == [16, 16, 16, 2, 1] and eng.stats.prefill_portions == 4


def test_eos_is_emitted_and_counted():
    """jllm/engine/engine.py:507-512."""
    prompt = [5, 6, 7]
    full = expected(prompt, 10)
    eos = full[3]
    eng, _ = make(block_size=4, max_model_len=64)
    got = eng.generate([prompt], SamplingParams(max_new_tokens=10, eos_id=eos))
    assert got == [full[:full.index(eos) + 1]]


def test_fifo_admission_slots_and_arrival_steps():
    eng, core = make(block_size=4, max_num_seqs=2, max_model_len=64, max_num_batched_tokens=64)
    ids = [eng.add_request([i, i + 1, i + 2], SamplingParams(max_new_tokens=2), arrival_step=s)
           for i, s in ((10, 0), (20, 0), (30, 0), (40, 6))]
    drain(eng)
    first_seen = {}
    for i, s in enumerate(core.steps):
        for rid, *_ in s:
            first_seen.setdefault(rid, i)
    assert first_seen[ids[0]] == first_seen[ids[1]] == 0      # two slots
    assert first_seen[ids[2]] == 2                            # a slot frees after two tokens each
    assert first_seen[ids[3]] >= 4                            # not before its arrival step (idle steps run nothing)
    assert eng.scheduler.step_index >= 7


def test_prefix_cache_decisions():
    """Adapted from the reference's tests/test_engine.py:83-126, 189-227 and
    tests/test_scheduler.py:166-243: with 'the last prompt token is always computed' a repeated
    32-token prompt hits 1 page of 2 and recomputes the other; a prompt sharing only the first
    page hits exactly 1."""
    eng, core = make(block_size=16, max_num_seqs=2, max_model_len=128, max_num_batched_tokens=64)
    prompt = list(range(32))
    first = eng.generate([prompt], SamplingParams(max_new_tokens=4))
    assert eng.stats.cache_hit_blocks == 0
    second = eng.generate([prompt], SamplingParams(max_new_tokens=4))
    assert second == first and eng.stats.cache_hit_blocks == 1 and eng.stats.cache_hit_tokens == 16
    assert core.steps[-4][0][1:3] == (16, 16)                 # only the last 16 tokens were run
    other = prompt[:16] + [90] * 10
    eng.generate([other], SamplingParams(max_new_tokens=2))
    assert eng.stats.cache_hit_blocks == 2
    # a cached and a cold request admitted together: one step holds the cold prompt whole and the
    # cached one's remainder; generated tokens enter the cache as pages fill (engine.py:476-490)
    n0 = len(core.steps)
    eng.generate([prompt, [50] * 20], SamplingParams(max_new_tokens=1))
    assert [(c, n) for _, c, n, _ in core.steps[n0]] == [(16, 16), (0, 20)]
    assert eng.stats.cache_hit_blocks == 3
    long = eng.generate([prompt], SamplingParams(max_new_tokens=20))[0]
    again = eng.generate([prompt + long[:17]], SamplingParams(max_new_tokens=1))
    assert core.steps[-1][0][1] == 48 and again == [expected(prompt + long[:17], 1)]


def test_a_request_waits_for_pages_that_a_running_request_is_computing():
    """Four prompts arrive together; two share their first 64 tokens.  The second of the two is
    put off until the first has computed the shared pages, takes them over, and the ones behind it
    are admitted meanwhile.  Tokens are what they are without the prefix cache."""
    kw = dict(block_size=16, max_num_seqs=4, max_model_len=256, max_num_batched_tokens=96, max_chunk=32)
    shared = list(range(64))
    prompts = [shared + [70 + i for i in range(20)], shared + [80] * 9, [5] * 40, [6] * 33]
    eng, core = make(**kw)
    got = eng.generate(prompts, SamplingParams(max_new_tokens=3))
    assert got == [expected(p, 3) for p in prompts]
    first_step = {rid: i for i, log in reversed(list(enumerate(core.steps))) for rid, *_ in log}
    ids = sorted(first_step)                                   # request ids in order of arrival
    assert first_step[ids[0]] == 0 and first_step[ids[2]] == 0 and first_step[ids[3]] == 0
    assert first_step[ids[1]] == 2                             # after two 32-token portions of the first
    start = [log for log in core.steps[2] if log[0] == ids[1]][0]
    assert start[1] == 64                                      # it begins behind the pages it took over
    assert eng.stats.cache_hit_blocks == 4 and eng.stats.prefix_waits == 2
    plain, _ = make(enable_prefix_cache=False, **kw)
    assert plain.generate(prompts, SamplingParams(max_new_tokens=3)) == got
    assert plain.stats.prefix_waits == 0 and plain.stats.cache_hit_blocks == 0
    # the sharer does not wait for a request that has its prompt behind it already
    eng2, _ = make(**kw)
    eng2.generate([prompts[0]], SamplingParams(max_new_tokens=1))
    eng2.generate([prompts[1]], SamplingParams(max_new_tokens=1))
    assert eng2.stats.prefix_waits == 0 and eng2.stats.cache_hit_blocks == 4


def test_requests_that_can_never_fit_are_refused():
    eng, _ = make(block_size=4, max_num_seqs=2, max_model_len=64, max_prefill_len=32, num_blocks=1 + 5)
    with pytest.raises(ValueError, match="empty prompt"):
        eng.add_request([])
    with pytest.raises(ValueError, match="max_prefill_len=32"):
        eng.add_request([1] * 33)
    with pytest.raises(ValueError, match="max_model_len"):
        eng.add_request([1] * 30, SamplingParams(max_new_tokens=40))
    with pytest.raises(ValueError, match="needs 6 pages"):
        eng.add_request([1] * 20, SamplingParams(max_new_tokens=4))
    with pytest.raises(ValueError, match="vocabulary"):
        eng.add_request([VOCAB])
    eng.add_request([1] * 16, SamplingParams(max_new_tokens=4))       # exactly 5 pages: accepted
    assert drain(eng)


def test_decode_without_a_page_preempts_the_newest_request():
    # 6 pages of 4: two requests of 9 prompt tokens take 3 pages each (12 slots, 9 used); after 3
    # decoded tokens each needs a 4th page and none is free
    eng, core = make(block_size=4, max_num_seqs=2, max_model_len=64, max_num_batched_tokens=64, num_blocks=1 + 6,
                     enable_prefix_cache=False)
    p0, p1 = list(range(9)), list(range(20, 29))
    a = eng.add_request(p0, SamplingParams(max_new_tokens=8))
    b = eng.add_request(p1, SamplingParams(max_new_tokens=8))
    ra, rb = eng.requests[a], eng.requests[b]
    drain(eng)
    assert eng.stats.preemptions >= 1
    assert rb.num_preemptions >= 1 and ra.num_preemptions == 0   # the newest yields
    assert ra.output_ids == expected(p0, 8) and rb.output_ids == expected(p1, 8)
    # the preempted request was recomputed from position 0: prompt and the tokens it had generated
    restarts = [s for s in core.steps for rid, c, n, _ in s if rid == b and c == 0]
    assert len(restarts) >= 2
    assert core.cache.num_free_pages() == 6


def test_prompt_portion_is_shortened_or_postponed_when_pages_are_short():
    eng, core = make(block_size=4, max_num_seqs=2, max_model_len=64, max_num_batched_tokens=64, num_blocks=1 + 6,
                     enable_prefix_cache=False)
    a = eng.add_request(list(range(14)), SamplingParams(max_new_tokens=2))     # 4 pages
    b = eng.add_request(list(range(30, 44)), SamplingParams(max_new_tokens=2))  # wants 4, only 2 are free
    ra, rb = eng.requests[a], eng.requests[b]
    drain(eng)
    assert core.steps[0] == [(a, 0, 14, [13])]                # b is not admitted: its first portion has no room
    assert ra.output_ids == expected(list(range(14)), 2)
    assert rb.output_ids == expected(list(range(30, 44)), 2)
    assert eng.stats.preemptions == 0


def test_lone_request_larger_than_the_free_pages_starts_with_what_fits():
    eng, core = make(block_size=4, max_num_seqs=2, max_model_len=64, max_num_batched_tokens=64, num_blocks=1 + 6,
                     max_chunk=64, enable_prefix_cache=False)
    eng.add_request(list(range(22)), SamplingParams(max_new_tokens=2))          # 6 pages at full length
    drain(eng)
    assert sum(n for s in core.steps for _, _, n, _ in s) == 22 + 1


def test_baseline_workload_b_under_a_24_token_budget():
    """5 requests, prompts 1/9/40/64/100 (two share a 32-token prefix), arrivals at steps
    0, 0, 2, 3, 5, budget 24, 20 new tokens each."""
    rng = np.random.default_rng(7)
    shared = rng.integers(0, VOCAB, size=32).tolist()
    prompts = [rng.integers(0, VOCAB, size=1).tolist(), rng.integers(0, VOCAB, size=9).tolist(),
               shared + rng.integers(0, VOCAB, size=8).tolist(), shared + rng.integers(0, VOCAB, size=32).tolist(),
               rng.integers(0, VOCAB, size=100).tolist()]
    eng, core = make(block_size=16, max_num_seqs=4, max_model_len=128, max_num_batched_tokens=24)
    got = eng.generate(prompts, SamplingParams(max_new_tokens=20, temperature=0.8, seed=7), arrival_steps=[0, 0, 2, 3, 5])
    assert got == [expected(p, 20) for p in prompts]
    assert all(sum(n for _, _, n, _ in s) <= 24 for s in core.steps)
    mixed = [s for s in core.steps if any(n > 1 for _, _, n, _ in s) and any(n == 1 and c > 0 for _, c, n, _ in s)]
    assert mixed, "prompt portions never ran beside decoded tokens"
    # the second sharer arrives one step after the first, when only the first common page is full:
    # it waits one step for the second and takes both over
    assert eng.stats.cache_hit_blocks == 2 and eng.stats.prefix_waits == 1


@pytest.mark.parametrize("seed", range(4))
def test_random_workloads_with_few_pages_finish_right(seed):
    rng = np.random.default_rng(seed)
    n = 12
    prompts = [rng.integers(0, 5, size=int(rng.integers(1, 40))).tolist() for _ in range(n)]
    new = [int(rng.integers(1, 16)) for _ in range(n)]
    eng, core = make(block_size=4, max_num_seqs=int(rng.integers(1, 5)), max_model_len=64,
                     max_num_batched_tokens=int(rng.integers(2, 30)), num_blocks=1 + int(rng.integers(14, 24)))
    got = eng.generate(prompts, [SamplingParams(max_new_tokens=k) for k in new],
                       arrival_steps=sorted(int(x) for x in rng.integers(0, 30, size=n)))
    assert got == [expected(p, k) for p, k in zip(prompts, new)]
    core.cache.check_invariants()
    assert core.cache.num_free_pages() == eng.config.usable_pages


def test_the_stepped_loop_hands_out_finished_requests_and_keeps_none():
    """The reference's canonical loop (tests/_greedy.py:34-43 there): add_request, then step while
    has_work, collecting events.  Every request's last event says finished and carries the
    request; the engine's own table holds waiting and running requests only, so a long-lived
    engine does not grow with the requests it has served."""
    prompts = [[1, 2, 3], list(range(40)), [7] * 17, [9], list(range(50, 70))]
    eng, core = make(max_num_seqs=2, max_model_len=128, block_size=8, max_num_batched_tokens=16)
    rids = [eng.add_request(p, SamplingParams(max_new_tokens=5 + i)) for i, p in enumerate(prompts)]
    assert sorted(eng.requests) == rids
    tokens, done, peak = {r: [] for r in rids}, {}, 0
    while eng.has_work():
        for ev in eng.step():
            assert ev.request_id not in done
            tokens[ev.request_id].append(ev.token)
            assert (ev.request is not None) == ev.finished
            if ev.finished:
                done[ev.request_id] = ev.request
                assert ev.request_id not in eng.requests
        peak = max(peak, len(eng.requests))
    assert eng.requests == {} and sorted(done) == rids
    for i, (rid, p) in enumerate(zip(rids, prompts)):
        assert tokens[rid] == done[rid].output_ids == expected(p, 5 + i) and done[rid].prompt_ids == p
    core.cache.check_invariants()
    assert core.cache.num_free_pages() == eng.config.usable_pages


# ------------------------------------------------------------------ a decode step started ahead of the tokens
class FakeDrawn:
    def __init__(self, tokens):
        self.tokens, self.rows = list(tokens), len(tokens)


class FakeAhead:
    """What the GPU engine hands the loop so that a decode step can follow the one before it: here
    on the host, with the same duties towards the cache manager (pages reserved at the start of the
    step, the token committed once the loop knows it)."""

    def __init__(self, core, refuse_every=0):
        self.core, self.refuse_every = core, refuse_every
        self.asked = self.followed = 0
        self.committed = []

    @staticmethod
    def launch(rows, temps, keys):
        assert len(rows) == len(temps) == len(keys)
        return FakeDrawn(rows)

    @staticmethod
    def finish(drawn):
        return drawn.tokens

    def follow(self, request_ids, drawn):
        cache = self.core.cache
        self.asked += 1
        if self.refuse_every and self.asked % self.refuse_every == 0:
            return None                                  # as if that step had not been captured yet
        promised = [0] * len(cache.groups)
        for r in request_ids:
            if not cache.can_store(r, 1, reserve=promised):
                return None
            promised = [p + n for p, n in zip(promised, cache.pages_needed(r, 1))]
        rows, log = [], []
        for k, r in enumerate(request_ids):
            cache.reserve(r, 1)
            ctx = cache.requests[r].tokens
            log.append((r, len(ctx), 1, [0]))
            rows.append(next_token(ctx + [drawn.tokens[k]]))
        self.core.steps.append(log)
        self.followed += 1
        return rows

    def commit(self, request_id, token):
        self.committed.append((request_id, token))
        self.core.cache.commit(request_id, [token])
        self.core.cache.check_invariants()


def make_ahead(refuse_every=0, **kw):
    cfg = EngineConfig(**kw)
    core = FakeCore(cfg)
    ahead = FakeAhead(core, refuse_every)
    return Engine(cfg, core.cache, core.run, core.sample, VOCAB, ahead=ahead), core, ahead


@pytest.mark.parametrize("seed", range(6))
def test_steps_started_ahead_change_nothing_that_a_caller_sees(seed):
    """The same requests through the loop with and without decode steps started ahead: the events
    of every call of ``step`` are the same (a step started ahead may hold a row more, of a request
    that ended on its eos_id in the step before)."""
    rng = np.random.default_rng(100 + seed)
    n = 7
    prompts = [rng.integers(0, 5, size=int(rng.integers(1, 30))).tolist() for _ in range(n)]
    params = [SamplingParams(max_new_tokens=int(rng.integers(1, 24)), eos_id=int(rng.integers(0, VOCAB)) if i % 2 else None)
              for i in range(n)]
    kw = dict(block_size=4, max_num_seqs=n if seed % 2 else int(rng.integers(2, 6)), max_model_len=64,
              max_num_batched_tokens=int(rng.integers(8, 40)), num_blocks=1 + int(rng.integers(20, 40)))
    logs = []
    for refuse in (None, 0, 3):
        if refuse is None:
            eng, core = make(**kw)
            ahead = None
        else:
            eng, core, ahead = make_ahead(refuse, **kw)
        for p, sp in zip(prompts, params):
            eng.add_request(p, sp)
        events = [[(e.request_id, e.token, e.finished) for e in step] for step in drain(eng)]
        core.cache.check_invariants()
        assert core.cache.num_free_pages() == eng.config.usable_pages and not core.cache.requests
        per_request = {}
        for step in events:
            for r, t, _ in step:
                per_request.setdefault(r, []).append(t)
        # with a slot for everybody nobody ever waits and every call gives the same events; otherwise a request
        # that waits for the slot of one that ends on its eos_id is admitted one step later
        logs.append((per_request, eng.stats.emitted_tokens, events if seed % 2 else None))
        if ahead is not None and seed % 2:
            assert ahead.followed > 0
    assert logs[0] == logs[1] == logs[2]
    assert logs[0][0] == {i: expected(p, sp.max_new_tokens, sp.eos_id) for i, (p, sp) in enumerate(zip(prompts, params))}


def test_a_step_is_started_ahead_only_when_the_next_one_is_known():
    eng, core, ahead = make_ahead(block_size=4, max_num_seqs=2, max_model_len=64, max_num_batched_tokens=32)
    a = eng.add_request([1, 2, 3], SamplingParams(max_new_tokens=4))
    b = eng.add_request([4, 5], SamplingParams(max_new_tokens=6))
    c = eng.add_request([6], SamplingParams(max_new_tokens=5))           # waits for a slot
    eng.step()                                                            # prompts of a and b: nothing to follow
    assert ahead.asked == 0 and eng._under_way is None
    eng.step()                                                            # decodes; c waits, but every slot is taken: followed
    assert ahead.asked == 1 and eng._under_way is not None
    eng.step()                                                            # the step under way, and the one after it
    assert ahead.asked == 2
    eng.step()                                                            # a's last token (4): the next step is another one
    assert a not in eng.requests and ahead.asked == 2 and eng._under_way is None
    eng.step()                                                            # b decodes beside c's prompt
    assert ahead.asked == 2
    eng.step()                                                            # b's last token: not followed either
    assert b not in eng.requests and ahead.asked == 2
    eng.step()                                                            # c alone, its third token of five: followed
    assert ahead.asked == 3 and eng._under_way is not None
    events = eng.step()                                                   # the step under way, and one more after it
    assert [(e.request_id, e.finished) for e in events] == [(c, False)] and ahead.asked == 4
    events = eng.step()                                                   # c's last token: nothing follows
    assert [(e.request_id, e.finished) for e in events] == [(c, True)] and ahead.asked == 4
    assert not eng.has_work() and eng._under_way is None
    assert core.cache.num_free_pages() == eng.config.usable_pages
    assert events[0].request.output_ids == expected([6], 5)
    # a free slot and somebody waiting for it: the next step is not known
    d = eng.add_request([7, 8], SamplingParams(max_new_tokens=6))
    eng.step(), eng.step()
    assert eng._under_way is not None
    e = eng.add_request([9], SamplingParams(max_new_tokens=2))
    eng.step()
    assert eng._under_way is None and d in eng.requests and e in eng.requests


def test_a_request_that_ends_on_its_eos_leaves_a_row_of_the_step_under_way_unused():
    prompts = [[1, 2, 3], [4, 5, 6, 7]]
    want = [expected(p, 12) for p in prompts]
    eos = want[0][3]                                  # the first request ends with its 4th token ...
    assert eos not in want[0][:3], "pick another prompt"
    eng, core, ahead = make_ahead(block_size=4, max_num_seqs=2, max_model_len=64, max_num_batched_tokens=32)
    a = eng.add_request(prompts[0], SamplingParams(max_new_tokens=12, eos_id=eos))
    b = eng.add_request(prompts[1], SamplingParams(max_new_tokens=12))
    out = {a: [], b: []}
    ended_at = None
    for call in range(40):
        if not eng.has_work():
            break
        for e in eng.step():
            out[e.request_id].append(e.token)
            if e.request_id == a and e.finished:
                ended_at = call
                assert eng._under_way is not None     # ... while the step after it was already started with a row for it
                assert [i.request.request_id for i in eng._under_way.items] == [a, b]
    assert out[a] == want[0][:4] and out[b] == want[1] and ended_at is not None
    assert all(r != a or t != eos for r, t in ahead.committed)           # its last token was never committed: it had ended
    assert core.cache.num_free_pages() == eng.config.usable_pages and not core.cache.requests


def test_abort_with_a_step_under_way():
    eng, core, ahead = make_ahead(block_size=4, max_num_seqs=2, max_model_len=64, max_num_batched_tokens=32)
    eng.add_request([1, 2, 3], SamplingParams(max_new_tokens=10))
    eng.step(), eng.step()
    assert eng._under_way is not None
    eng.abort_all()
    assert eng._under_way is None and not eng.has_work()
    assert core.cache.num_free_pages() == eng.config.usable_pages
    assert eng.generate([[5, 6]], SamplingParams(max_new_tokens=5)) == [expected([5, 6], 5)]


@pytest.mark.parametrize("with_ahead", [False, True])
def test_a_step_whose_tokens_cannot_be_chosen_ends_its_requests_and_nothing_else(with_ahead):
    """The sampler raises for a row of logits without a maximum.  By then the cache holds the
    step's tokens and a step started ahead may hold a page more: the loop ends the requests of that
    step (everything they hold goes back), raises, and serves later requests as if nothing had
    happened."""
    kw = dict(block_size=4, max_num_seqs=2, max_model_len=64, max_num_batched_tokens=32)
    eng, core, ahead = make_ahead(**kw) if with_ahead else (*make(**kw), None)
    fail_at = {"calls": 0}

    def failing(fn):
        def wrapped(arg, *more):
            fail_at["calls"] += 1
            if fail_at["calls"] == 4:
                raise FloatingPointError("logits row(s) [0] of 1 hold no finite maximum")
            return fn(arg, *more)
        return wrapped

    if with_ahead:
        ahead.finish = failing(ahead.finish)
    else:
        eng._sample = failing(eng._sample)
    a = eng.add_request([1, 2, 3], SamplingParams(max_new_tokens=10))
    got = []
    with pytest.raises(FloatingPointError):
        for _ in range(10):
            got += [e.token for e in eng.step()]
    assert got == expected([1, 2, 3], 3)
    assert a not in eng.requests and not eng.has_work() and eng._under_way is None
    core.cache.check_invariants()
    assert core.cache.num_free_pages() == eng.config.usable_pages and not core.cache.requests
    assert eng.generate([[5, 6]], SamplingParams(max_new_tokens=5)) == [expected([5, 6], 5)]
