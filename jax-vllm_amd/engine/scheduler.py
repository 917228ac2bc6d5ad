"""Continuous-batching scheduler: admits requests, cuts prompts into portions under a token
budget, decodes, finishes and frees, and decides what happens when pages run out.

Reference: ``jllm/engine/engine.py:161-168, 282-512``.  Kept: FIFO admission into at most
``max_num_seqs`` slots (a request that would share pages which a running request is still
computing waits for them and lets the ones behind it pass), prefix-cache lookup at admission, a request's first token comes from
the step that ends its prompt, finish on ``max_new_tokens`` or on an emitted ``eos_id``,
release at finish.  Changed: one mixed batch per step under ``max_num_batched_tokens``
(decode tokens first, then prompt portions of any length) instead of one block per
prefilling request plus a separate decode call; and the pool may be smaller than the worst
case, which the reference refuses (``engine.py:89-94``).

When pages run out:
  * a request is admitted only if its first portion's pages are free;
  * a prompt portion is shortened to the pages that are free, or postponed to a later step;
  * a decode that needs a page and finds none preempts the most recently admitted running
    request (possibly itself): its pages are given back (hashed full pages stay revivable),
    it returns to the head of the waiting queue and is recomputed, prompt and tokens
    generated so far, when it is admitted again;
  * if nothing at all could be scheduled while requests are running, the most recently
    admitted one is preempted so that the others can advance;
  * a request that could never fit the pool is refused when it is added.

The scheduler is host logic only: it sees the cache manager's counts, never the device.
"""
from __future__ import annotations

from collections import deque
from dataclasses import dataclass, field
from typing import Optional

from ..config.engine import EngineConfig
from .request import EngineStats, Request


@dataclass
class ScheduledItem:
    request: Request
    num_tokens: int            # tokens of request.all_tokens[num_computed:] to run in this step
    samples: bool              # the portion reaches the end: a token is sampled from its last logits


@dataclass
class SchedulerOutput:
    items: list = field(default_factory=list)
    preempted: list = field(default_factory=list)

    @property
    def num_tokens(self) -> int:
        return sum(i.num_tokens for i in self.items)


class Scheduler:
    def __init__(self, config: EngineConfig, cache, stats: Optional[EngineStats] = None):
        """``cache``: the cache manager (``start``, ``finish``, ``can_store``, ``pages_needed``,
        ``groups``)."""
        self.config, self.cache = config, cache
        self.stats = stats or EngineStats()
        self.waiting: deque = deque()
        self.running: list = []          # in order of admission
        self.step_index = 0
        self._admissions = 0

    # ---- queue
    def add(self, request: Request) -> None:
        cfg = self.config
        n = len(request.prompt_ids)
        if n == 0:
            raise ValueError("empty prompt")
        if n > cfg.prompt_limit:
            raise ValueError(f"prompt too long for max_prefill_len={cfg.prompt_limit}")
        if n + request.sampling.max_new_tokens > cfg.max_model_len:
            raise ValueError("prompt+max_new exceeds max_model_len")
        total_pages = -(-(n + request.sampling.max_new_tokens) // cfg.page_size)
        for g in self.cache.groups:
            if g.window is None and total_pages > g.pool.num_pages:
                raise ValueError(
                    f"request needs {total_pages} pages at full length, the pool has {g.pool.num_pages}"
                )
        self.waiting.append(request)

    def has_work(self) -> bool:
        return bool(self.waiting) or bool(self.running)

    # ---- one scheduling decision
    def schedule(self) -> SchedulerOutput:
        cfg, cache = self.config, self.cache
        out = SchedulerOutput()
        budget = cfg.max_num_batched_tokens
        reserved = [0] * len(cache.groups)
        self.stats.scheduler_loops += 1

        def take(req, n):
            need = cache.pages_needed(req.request_id, n)
            for g in range(len(reserved)):
                reserved[g] += need[g]

        def fits(need):
            return all(g.pool.num_free - r >= n for g, n, r in zip(cache.groups, need, reserved))

        # 1. decodes (one token each), oldest first; a decode without a page preempts the newest
        preempted_any = False
        for req in list(self.running):
            if budget <= 0:
                break
            if req.num_remaining != 1 or (preempted_any and req not in self.running):
                continue
            need = cache.pages_needed(req.request_id, 1)
            while not fits(need):
                victim = self._newest_unscheduled(out)
                if victim is None:
                    break
                self._preempt(victim, out)
                preempted_any = True
                if victim is req:
                    break
            if (not preempted_any or req in self.running) and fits(need):
                for g in range(len(reserved)):
                    reserved[g] += need[g]
                out.items.append(ScheduledItem(req, 1, True))
                budget -= 1

        # 2. portions of prompts (or of recomputation) of running requests, oldest first
        for req in self.running:
            if req.num_remaining <= 1 or budget <= 0:
                continue
            n = self._fit_portion(req, min(req.num_remaining, cfg.chunk_limit, budget), reserved)
            if n > 0:
                take(req, n)
                out.items.append(ScheduledItem(req, n, n == req.num_remaining))
                budget -= n

        # 3. admission, FIFO; a request whose leading pages a running request is about to compute
        #    waits until they are there (it then takes them over instead of computing them again)
        at = 0
        while at < len(self.waiting) and budget > 0 and len(self.running) < cfg.max_num_seqs:
            req = self.waiting[at]
            if req.arrival_step > self.step_index or req in out.preempted:
                break
            if self._waits_for_prefix(req):
                self.stats.prefix_waits += 1
                at += 1
                continue
            tokens = req.all_tokens
            cached = cache.start(req.request_id, tokens)
            n = min(len(tokens) - cached, cfg.chunk_limit, budget)
            if not cache.can_store(req.request_id, n, reserve=reserved):
                # alone in the engine nothing else will ever free pages: start with what fits
                n = self._fit_portion(req, n, reserved, cached) if not self.running else 0
                if n <= 0:
                    cache.finish(req.request_id)     # gives the hit pages back untouched
                    break
            del self.waiting[at]
            req.num_computed = cached
            req.slot = cache.slot(req.request_id)
            req.admitted_order = self._admissions
            self._admissions += 1
            self.running.append(req)
            self.stats.admissions += 1
            self.stats.cache_hit_blocks += cached // cfg.page_size
            self.stats.cache_hit_tokens += cached
            take(req, n)
            out.items.append(ScheduledItem(req, n, n == req.num_remaining))
            budget -= n

        # 4. nothing runs although requests hold pages: free the newest so the rest can move
        if not out.items and self.running:
            self._preempt(self.running[-1], out)
            return self.schedule() if self.running or self._arrived() else out

        self.step_index += 1
        return out

    def _waits_for_prefix(self, req: Request) -> bool:
        """Whether a running request is still computing full pages whose tokens are the leading
        tokens of ``req`` too (pages are found by their content once they are full)."""
        if not getattr(self.cache, "prefix_cache", False):
            return False
        ps = self.config.page_size
        tokens = req.all_tokens
        limit = (len(tokens) - 1) // ps            # the page of the last token is never taken over
        if limit == 0:
            return False
        first = tokens[:ps]
        for other in self.running:
            if other.num_remaining <= 1:
                continue
            theirs = other.all_tokens
            if theirs[:ps] != first:
                continue
            n = 1
            while n < limit and len(theirs) >= (n + 1) * ps and theirs[n * ps:(n + 1) * ps] == tokens[n * ps:(n + 1) * ps]:
                n += 1
            if other.num_computed < n * ps:
                return True
        return False

    def _arrived(self) -> bool:
        return bool(self.waiting) and self.waiting[0].arrival_step <= self.step_index

    def _fit_portion(self, req, n, reserved, context_len=None) -> int:
        """The largest portion <= n whose pages are free now (0: postponed)."""
        cache = self.cache
        if cache.can_store(req.request_id, n, reserve=reserved):
            return n
        self.stats.stalled_portions += 1
        ps = self.config.page_size
        rc_len = cache.context_len(req.request_id) if context_len is None else context_len
        # tokens that fit into the pages the request already holds plus the free ones
        free = min(g.pool.num_free - r for g, r in zip(cache.groups, reserved))
        held = min(len(cache.block_table(req.request_id, g)) for g in range(len(cache.groups)))
        room = (held + max(free, 0)) * ps - rc_len
        m = max(0, min(n, room))
        while m > 0 and not cache.can_store(req.request_id, m, reserve=reserved):
            m -= 1
        return m

    def _newest_unscheduled(self, out) -> Optional[Request]:
        scheduled = {id(i.request) for i in out.items}
        for req in reversed(self.running):
            if id(req) not in scheduled:
                return req
        return None

    def _preempt(self, req: Request, out: SchedulerOutput) -> None:
        self.cache.finish(req.request_id)
        self.running.remove(req)
        req.num_computed = 0
        req.slot = None
        req.num_preemptions += 1
        self.stats.preemptions += 1
        self.waiting.appendleft(req)
        out.preempted.append(req)

    # ---- after the step ran
    def advance(self, item: ScheduledItem, new_token: Optional[int]) -> bool:
        """Record that the item's tokens are computed; with a sampled token, append it and decide
        whether the request is finished (``max_new_tokens`` reached or ``eos_id`` emitted, which
        is itself counted: ``jllm/engine/engine.py:507-512``).  Returns finished."""
        req = item.request
        req.num_computed += item.num_tokens
        if new_token is None:
            return False
        req.output_ids.append(int(new_token))
        sp = req.sampling
        done = len(req.output_ids) >= sp.max_new_tokens or (sp.eos_id is not None and new_token == sp.eos_id)
        if done:
            self.finish(req)
        return done

    def finish(self, req: Request) -> None:
        req.finished = True
        req.slot = None
        self.running.remove(req)
        self.cache.finish(req.request_id)
