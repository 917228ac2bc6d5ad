"""Request-level types.  Reference: ``jllm/engine/request.py`` (``SamplingParams`` with
``max_new_tokens=64`` and ``eos_id``, ``Request``, ``StepEvent``, ``EngineStats``).  Added:
temperature and seed (the reference's HTTP schemas carry a temperature that is never read,
``jllm/server.py:42,50``), an arrival step, and counters for budgets, pages and preemption.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Optional


@dataclass
class SamplingParams:
    max_new_tokens: int = 64
    eos_id: Optional[int] = None
    temperature: float = 0.0          # 0: greedy (argmax, lowest index on ties)
    seed: Optional[int] = None        # None: the engine's seed combined with the request id


@dataclass(eq=False)   # requests are compared by identity: queue membership tests stay O(1) per item
class Request:
    request_id: int
    prompt_ids: list
    sampling: SamplingParams
    output_ids: list = field(default_factory=list)
    finished: bool = False
    slot: Optional[int] = None
    arrival_step: int = 0             # first scheduler step at which it may be admitted
    num_computed: int = 0             # tokens of prompt+output whose keys/values are in the cache
    num_preemptions: int = 0
    admitted_order: int = -1

    @property
    def all_tokens(self) -> list:
        return self.prompt_ids + self.output_ids

    @property
    def num_remaining(self) -> int:
        """Tokens still to be run before the next token can be sampled."""
        return len(self.prompt_ids) + len(self.output_ids) - self.num_computed


@dataclass
class StepEvent:
    request_id: int
    token: int
    finished: bool
    request: Optional[Request] = None   # with the finishing event only: the engine lets go of it there


@dataclass
class EngineStats:
    admissions: int = 0
    scheduler_loops: int = 0          # decisions of the scheduler (a decode step started ahead of its tokens needs none)
    steps_run: int = 0                # steps that ran at least one token
    prefill_tokens: int = 0           # prompt (or recomputed) tokens run
    decode_tokens: int = 0            # single decoded tokens run
    prefill_portions: int = 0         # the reference's extend_calls
    decode_calls: int = 0
    emitted_tokens: int = 0
    cache_hit_blocks: int = 0
    cache_hit_tokens: int = 0
    preemptions: int = 0
    stalled_portions: int = 0         # portions shortened or postponed for lack of pages
    prefix_waits: int = 0             # admissions put off until a running request had computed shared pages
    max_batched_tokens: int = 0
    graph_replays: int = 0
    steps_ahead: int = 0              # decode steps started before the tokens of the step before were on the host
