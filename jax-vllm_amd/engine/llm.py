"""The Python entry point: an engine object with ``add_request / step / has_work`` and a
blocking ``generate``, plus module-level functions in the reference's own manner
(``make_driver``, ``add_request(driver, ...)``, ``step(driver)``, ``has_work(driver)``,
``prewarm``: ``jllm/engine/engine.py:63-208``; the canonical loop is
``tests/_greedy.py:34-43``).  The engine is stepped by its caller, in the caller's thread;
the reference's background thread and per-request queues belong to its server and are not
built.  Tokens in, tokens out: tokenisers are not part of the engine.
"""
from __future__ import annotations

from pathlib import Path
from typing import Mapping, Optional, Sequence, Union

from ..config.engine import EngineConfig
from ..sampling.keys import draw_key
from .entries import StepEntry
from .request import EngineStats, Request, SamplingParams, StepEvent
from .scheduler import ScheduledItem, Scheduler


class _StepUnderWay:
    """A decode step that is already on the GPU: its items, and its tokens being chosen."""

    def __init__(self, items: list, drawn):
        self.items, self.drawn = items, drawn


class Engine:
    """The host loop above the step function: requests in, ``StepEvent``s out.  It needs a cache
    manager for the scheduler, a ``run(entries, borrow=True)`` that returns logits for the
    wanted places, and a ``sample(logits, temperatures, keys)``; the GPU engine passes the real
    ones, host-only tests pass stand-ins.

    ``ahead`` (optional; the GPU engine passes one): lets a decode step follow the one before it
    on the GPU without the host in between.  It has ``launch(logits, temperatures, keys)`` and
    ``finish(drawn)``, the two halves of ``sample``; ``follow(request_ids, drawn)``, which starts
    one more decode step of the same requests with each row's token taken from the device, or
    returns None; and ``commit(request_id, token)`` for the tokens of such a step once they are
    known.  While step k runs, ``step`` then already starts step k + 1 of the same requests,
    waits for the tokens of step k only afterwards and returns step k's events as ever; the
    next call finds its step under way.  Only a step of decodes of every running request is
    followed, with nobody waiting for a free slot, none of them at its last token and pages at
    hand; a request that ends on its ``eos_id`` has one row of the step under way for nothing,
    which is ignored (whoever waits for its slot is admitted one step later than otherwise)."""

    def __init__(self, config: EngineConfig, cache, run, sample, vocab_size: int, ahead=None):
        self.config = config
        self.stats = EngineStats()
        self.scheduler = Scheduler(config, cache, self.stats)
        self._run, self._sample = run, sample
        self._ahead = ahead
        self._under_way: Optional[_StepUnderWay] = None
        self.vocab_size = vocab_size
        self._next_id = 0
        self.requests: dict = {}     # waiting and running requests by id; a finished one leaves with its last event

    # ---- the reference's loop: add_request / has_work / step
    def add_request(self, prompt_ids: Sequence[int], sampling: Optional[SamplingParams] = None,
                    arrival_step: int = 0) -> int:
        sp = sampling or SamplingParams()
        for t in prompt_ids:
            if not 0 <= int(t) < self.vocab_size:
                raise ValueError(f"token id {t} outside the vocabulary [0, {self.vocab_size})")
        if sp.max_new_tokens < 1:
            raise ValueError("max_new_tokens must be at least 1")
        rid = self._next_id
        req = Request(request_id=rid, prompt_ids=[int(t) for t in prompt_ids], sampling=sp, arrival_step=arrival_step)
        self.scheduler.add(req)
        self._next_id += 1
        self.requests[rid] = req
        return rid

    def has_work(self) -> bool:
        return self.scheduler.has_work()

    def _draw_arguments(self, sampled: list, ahead_by: int = 0):
        temps = [i.request.sampling.temperature for i in sampled]
        keys = [
            draw_key(i.request.sampling.seed if i.request.sampling.seed is not None else self.config.seed,
                     i.request.request_id, len(i.request.output_ids) + ahead_by)
            for i in sampled
        ]
        return temps, keys

    def _count(self, items: list) -> None:
        for item in items:
            if item.num_tokens == 1 and item.samples and item.request.output_ids:
                self.stats.decode_tokens += 1
                self.stats.decode_calls += 1
            else:
                self.stats.prefill_tokens += item.num_tokens
                self.stats.prefill_portions += 1
        self.stats.steps_run += 1
        self.stats.max_batched_tokens = max(self.stats.max_batched_tokens, sum(i.num_tokens for i in items))

    def _may_follow(self, items: list) -> bool:
        """Whether the step after this one is known already: the same decodes again."""
        sch = self.scheduler
        if self._ahead is None or len(items) != len(sch.running):
            return False
        if sch.waiting and len(sch.running) < self.config.max_num_seqs:
            return False                     # somebody may be admitted (with every slot taken nobody is)
        return all(i.num_tokens == 1 and i.samples and i.request.output_ids
                   and len(i.request.output_ids) + 1 < i.request.sampling.max_new_tokens for i in items)

    def step(self) -> list:
        """One scheduler iteration: schedule, run the mixed batch, sample, finish.  Returns the
        ``StepEvent`` of every token emitted.  The event that finishes a request carries the
        request (prompt, output, counters); the engine keeps nothing of it afterwards."""
        under_way, self._under_way = self._under_way, None
        tokens = drawn = None
        if under_way is not None and any(not i.request.finished for i in under_way.items):
            # the step that the call before this one started: row k belongs to its k-th item; the rows of
            # requests that ended on their eos_id meanwhile are not looked at
            row_of = {id(i): k for k, i in enumerate(under_way.items)}
            items = [i for i in under_way.items if not i.request.finished]
            drawn = under_way.drawn
            self.scheduler.step_index += 1
        else:
            out = self.scheduler.schedule()
            if not out.items:
                return []
            items = out.items
            entries = []
            for item in items:
                req = item.request
                toks = req.all_tokens[req.num_computed:req.num_computed + item.num_tokens]
                entries.append(StepEntry(req.request_id, toks, [item.num_tokens - 1] if item.samples else []))
            logits = self._run(entries, borrow=True)
            sampled = [i for i in items if i.samples]
            row_of = {id(i): k for k, i in enumerate(sampled)}
            temps, keys = self._draw_arguments(sampled)
            if self._ahead is not None and sampled:
                drawn = self._ahead.launch(logits, temps, keys)
            else:
                try:
                    tokens = self._sample(logits, temps, keys)
                except Exception:
                    self._drop(items)
                    raise
        self._count(items)
        # the step after this one, if it is known already, goes to the GPU before this one's tokens are awaited
        following = None
        if drawn is not None and [row_of.get(id(i)) for i in items] == list(range(drawn.rows)) and self._may_follow(items):
            logits = self._ahead.follow([i.request.request_id for i in items], drawn)
            if logits is not None:
                nxt = [ScheduledItem(i.request, 1, True) for i in items]
                temps, keys = self._draw_arguments(nxt, ahead_by=1)
                following = _StepUnderWay(nxt, self._ahead.launch(logits, temps, keys))
        if drawn is not None:
            try:
                tokens = self._ahead.finish(drawn)
            except Exception:
                # a step started ahead has run on a token nobody can use: it is never looked at
                self._drop(items)
                raise
        events = []
        for item in items:
            tok = tokens[row_of[id(item)]] if item.samples else None
            finished = self.scheduler.advance(item, tok)
            if tok is not None:
                self.stats.emitted_tokens += 1
                events.append(StepEvent(item.request.request_id, int(tok), finished,
                                        item.request if finished else None))
            if finished:
                self.requests.pop(item.request.request_id, None)
        if following is not None:
            for item in following.items:     # the step under way has read these tokens from the device
                if not item.request.finished:
                    self._ahead.commit(item.request.request_id, item.request.output_ids[-1])
            self._under_way = following
        return events

    def _drop(self, items: list) -> None:
        """No token could be chosen for this step (a row of logits without a maximum): the cache
        already holds the step's tokens, the requests do not, so its requests end here and give back
        what they hold, also what a step started ahead has reserved; the others go on."""
        for item in items:
            req = item.request
            if not req.finished:
                self.scheduler.finish(req)
            self.requests.pop(req.request_id, None)

    def abort_all(self) -> None:
        """Drop every waiting and running request and give back what they hold."""
        self._under_way = None             # what it has on the GPU ends by itself and is never looked at
        self.scheduler.waiting.clear()
        for req in list(self.scheduler.running):
            self.scheduler.finish(req)
        self.requests.clear()

    # ---- blocking use
    def generate(self, prompts: Sequence[Sequence[int]],
                 sampling: Union[SamplingParams, Sequence[SamplingParams], None] = None,
                 arrival_steps: Optional[Sequence[int]] = None) -> list:
        """Generated token ids of every prompt, in the order given."""
        if sampling is None or isinstance(sampling, SamplingParams):
            sampling = [sampling or SamplingParams()] * len(prompts)
        arrival_steps = arrival_steps or [0] * len(prompts)
        reqs = [self.requests[self.add_request(p, s, a)] for p, s, a in zip(prompts, sampling, arrival_steps)]
        while self.has_work():
            self.step()
        return [list(r.output_ids) for r in reqs]


class _Ahead:
    """What ``Engine`` needs to let a decode step follow the one before it on the GPU."""

    def __init__(self, core, sampler):
        self.core, self.launch, self.finish = core, sampler.launch, sampler.finish
        self.commit = core.commit_decode

    def follow(self, request_ids, drawn):
        return self.core.follow_decode(request_ids, drawn.tokens)


class LLM(Engine):
    """One model on one GPU behind a continuous-batching scheduler.

    ``model`` is a model folder (``config.json`` + safetensors), or a ``config.json``-style
    dict for random weights drawn on the device from ``random_seed``, or an already bound
    ``DecoderModel``.  The other arguments are the fields of ``EngineConfig``; the reference's
    names (``max_num_seqs``, ``max_model_len``, ``max_prefill_len``, ``block_size``,
    ``num_blocks``, ``dtype`` = "bf16" | "fp32") keep their meaning.
    """

    def __init__(self, model, *, random_seed: int = 0, device="cuda", **engine_options):
        from ..parts.model import DecoderModel
        from ..sampling.sampler import Sampler
        from ..weights import load_model, random_model_on_device
        from .core import EngineCore

        config = EngineConfig(**engine_options)
        if isinstance(model, DecoderModel):
            self.model = model
        elif isinstance(model, Mapping):
            self.model, self.model_config = random_model_on_device(model, random_seed, config.dtype, device=device)
        else:
            self.model, self.model_config = load_model(Path(model), config.dtype, device)
        self.core = EngineCore(self.model, config)
        self.sampler = Sampler(self.core.device)
        super().__init__(config, self.core.cache, self.core.run, self.sampler.sample, self.core.vocab_size,
                         ahead=_Ahead(self.core, self.sampler) if config.decode_ahead else None)
        self._replays_before = 0     # replays of a prewarm are not the requests'
        self._followed_before = 0

    def step(self) -> list:
        events = super().step()
        self.stats.graph_replays = self.core.graph_replays - self._replays_before
        self.stats.steps_ahead = self.core.steps_followed - self._followed_before
        return events

    def prewarm(self) -> float:
        """Do now what the first requests would otherwise wait for, and return the seconds it took
        (``jllm/engine/engine.py:182-208`` compiles its step programs for every batch shape there):
        the kernel libraries this model needs are built or loaded, the library's matrix products
        are initialised by one prompt portion, and the decode step is captured for every batch
        bucket up to ``max_num_seqs`` at the smallest block-table width.  Only with no request
        waiting or running; request ids, statistics and the prefix index are as before afterwards."""
        import time

        import torch

        if self.has_work():
            raise RuntimeError("prewarm needs an engine without waiting or running requests")
        t0 = time.perf_counter()
        from .core import _batch_bucket

        tuning = self.config.tune_library and self.config.dtype == "bfloat16"
        if tuning:
            # The library's first guess is far off for 65..256 rows (8B sizes, 128 rows: down 66 us, timed choice 45;
            # qkv at 256 rows 40 against 28).  Its timing pass runs at the first (eager) call of a shape, here and
            # only here; it is switched off again below, so a shape first seen while serving takes the first guess.
            # Buffers take turns while it times (512 MB), or it would time weights that sit in the cache.
            import os
            import tempfile

            tunable = torch.cuda.tunable
            tunable.set_filename(os.path.join(tempfile.gettempdir(), f"jax_vllm_amd_tuned_{os.getuid()}.csv"))
            tunable.set_rotating_buffer_size(512)
            tunable.enable(True)
            tunable.tuning_enable(True)

        saved = (self.stats, self._next_id, self.core.cache.prefix_cache)
        self.core.cache.prefix_cache = False     # the warm-up prompts must not enter the prefix index
        self.stats = self.scheduler.stats = EngineStats()
        try:
            buckets = sorted({_batch_bucket(n) for n in range(1, self.config.max_num_seqs + 1)
                              if _batch_bucket(n) <= self.config.max_num_seqs} | {self.config.max_num_seqs})
            room = min(self.config.prompt_limit, self.config.max_model_len - 4, self.config.max_num_batched_tokens)
            first = True
            for b in buckets:
                n = max(1, min(room, 64)) if first else 1     # one real portion for the matrix library, then single tokens
                first = False
                self.generate([[0] * n] + [[0]] * (b - 1), SamplingParams(max_new_tokens=4))
        finally:
            if tuning:
                torch.cuda.tunable.tuning_enable(False)      # the choices made stay in use
            self.core.cache.prefix_cache = saved[2]
            self.stats, self._next_id = saved[0], saved[1]
            self.scheduler.stats = self.stats
            self._replays_before = self.core.graph_replays
            self._followed_before = self.core.steps_followed
        torch.cuda.synchronize()
        return time.perf_counter() - t0


# ---- the reference's functional spelling ------------------------------------------------
def make_driver(model, max_num_seqs: int, max_model_len: int, max_prefill_len: Optional[int] = None,
                block_size: int = 16, num_blocks: Optional[int] = None, dtype: str = "bf16", **more) -> LLM:
    """``jllm/engine/engine.py:63-109`` with the same argument names.  ``model``: folder, config
    dict or bound model.  ``num_blocks`` below the worst case is allowed here."""
    return LLM(model, max_num_seqs=max_num_seqs, max_model_len=max_model_len, max_prefill_len=max_prefill_len,
               block_size=block_size, num_blocks=num_blocks, dtype=dtype, **more)


def add_request(driver: LLM, prompt_ids, sampling: Optional[SamplingParams] = None) -> int:
    return driver.add_request(prompt_ids, sampling)


def has_work(driver: LLM) -> bool:
    return driver.has_work()


def step(driver: LLM) -> list:
    return driver.step()


def prewarm(driver: LLM) -> float:
    """``jllm/engine/engine.py:182-208``: seconds spent on what the first requests would wait for."""
    return driver.prewarm()
