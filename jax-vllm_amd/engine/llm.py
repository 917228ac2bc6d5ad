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
from .scheduler import Scheduler


class Engine:
    """The host loop above the step function: requests in, ``StepEvent``s out.  It needs a cache
    manager for the scheduler, a ``run(entries, borrow=True)`` that returns logits for the
    wanted places, and a ``sample(logits, temperatures, keys)``; the GPU engine passes the real
    ones, host-only tests pass stand-ins."""

    def __init__(self, config: EngineConfig, cache, run, sample, vocab_size: int):
        self.config = config
        self.stats = EngineStats()
        self.scheduler = Scheduler(config, cache, self.stats)
        self._run, self._sample = run, sample
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

    def step(self) -> list:
        """One scheduler iteration: schedule, run the mixed batch, sample, finish.  Returns the
        ``StepEvent`` of every token emitted.  The event that finishes a request carries the
        request (prompt, output, counters); the engine keeps nothing of it afterwards."""
        out = self.scheduler.schedule()
        if not out.items:
            return []
        entries, sampled = [], []
        for item in out.items:
            req = item.request
            tokens = req.all_tokens[req.num_computed:req.num_computed + item.num_tokens]
            entries.append(StepEntry(req.request_id, tokens, [item.num_tokens - 1] if item.samples else []))
            if item.samples:
                sampled.append(item)
            if item.num_tokens == 1 and item.samples and req.output_ids:
                self.stats.decode_tokens += 1
                self.stats.decode_calls += 1
            else:
                self.stats.prefill_tokens += item.num_tokens
                self.stats.prefill_portions += 1
        self.stats.steps_run += 1
        self.stats.max_batched_tokens = max(self.stats.max_batched_tokens, out.num_tokens)
        logits = self._run(entries, borrow=True)
        temps = [i.request.sampling.temperature for i in sampled]
        keys = [
            draw_key(i.request.sampling.seed if i.request.sampling.seed is not None else self.config.seed,
                     i.request.request_id, len(i.request.output_ids))
            for i in sampled
        ]
        tokens = self._sample(logits, temps, keys)
        events, k = [], 0
        for item in out.items:
            tok = None
            if item.samples:
                tok = tokens[k]
                k += 1
            finished = self.scheduler.advance(item, tok)
            if tok is not None:
                self.stats.emitted_tokens += 1
                events.append(StepEvent(item.request.request_id, int(tok), finished,
                                        item.request if finished else None))
            if finished:
                self.requests.pop(item.request.request_id, None)
        return events

    def abort_all(self) -> None:
        """Drop every waiting and running request and give back what they hold."""
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
        super().__init__(config, self.core.cache, self.core.run, self.sampler.sample, self.core.vocab_size)
        self._replays_before = 0     # replays of a prewarm are not the requests'

    def step(self) -> list:
        events = super().step()
        self.stats.graph_replays = self.core.graph_replays - self._replays_before
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
            self.core.cache.prefix_cache = saved[2]
            self.stats, self._next_id = saved[0], saved[1]
            self.scheduler.stats = self.stats
            self._replays_before = self.core.graph_replays
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
