"""The step function and what it stands on: a bound model, the cache manager, the device
memory of every layer.

One call of ``EngineCore.run`` takes a batch of (request, its next tokens): portions of
prompts beside single decoded tokens, cut anywhere.  It runs only those tokens, as one
flattened batch, against what earlier steps left in the cache, stores their keys and
values, and returns float logits at the places asked for.  The reference has two device
programs instead, a prefill of exactly one block per row and a decode of one token per
row, padded to bucket shapes (``jllm/engine/generate.py:112-143, 233-265``,
``jllm/engine/engine.py:317-496``); their per-row arguments (``pos_starts``, block tables,
``valid_tokens``, ``last_token_idx``, ``phys_blocks``, ``slot_in_block``) are what the
flattened arrays built here carry per token and per request.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Optional, Sequence

import numpy as np
import torch

from ..cache.manager import CacheManager
from ..cache.storage import allocate_memories, cache_bytes_per_token, group_keys_of, has_state
from ..config.engine import EngineConfig
from .entries import StepEntry
from ..parts.model import DecoderModel
from ..parts.spec import StepContext
from ..weights.loader import TORCH_DTYPES


def _bucket(n: int, floor: int = 1) -> int:
    """The next power of two at or above n (and at least ``floor``)."""
    b = floor
    while b < n:
        b *= 2
    return b


def _batch_bucket(n: int) -> int:
    """Rows of the captured decode step that serves n requests: powers of two up to 16 (a step's
    time hardly depends on the rows there), beyond that also the values half-way (24, 48, 96, ...):
    at most a third of the rows are padding."""
    b = _bucket(n)
    if b > 16 and n <= b // 4 * 3:
        return b // 4 * 3
    return b


class _DecodeGraph:
    """Fixed host and device buffers of one captured decode step and the graph itself."""

    def __init__(self, rb: int, widths: tuple, n_groups: int, device):
        names = [("tokens", rb), ("positions", rb), ("token_req", rb), ("cu", rb + 1), ("ctx", rb), ("slots", rb),
                 ("rows", rb)]
        names += [(f"slot_mapping{g}", rb) for g in range(n_groups)]
        names += [(f"table{g}", rb * widths[g]) for g in range(n_groups)]
        self.rb, self.widths, self.n_groups = rb, widths, n_groups
        self.offsets, at = {}, 0
        for name, size in names:
            self.offsets[name] = (at, at + size)
            at += size
        self.host_tensor = torch.zeros(at, dtype=torch.int32, pin_memory=True)
        self.host = self.host_tensor.numpy()
        a, b = self.offsets["token_req"]
        self.host[a:b] = np.arange(rb, dtype=np.int32)
        a, b = self.offsets["cu"]
        self.host[a:b] = np.arange(rb + 1, dtype=np.int32)
        a, b = self.offsets["rows"]
        self.host[a:b] = np.arange(rb, dtype=np.int32)
        self.row_signature = [[None] * rb for _ in range(n_groups)]   # the cache manager's table signature per row
        self.dev = torch.zeros(at, dtype=torch.int32, device=device)
        self.graph = None
        self.logits = None
        self.ctx = None
        self.copied = None   # event recorded after each upload of the pinned buffer

    def segment(self, host, name):
        a, b = self.offsets[name]
        return host[a:b]

    def dev_segment(self, name):
        a, b = self.offsets[name]
        return self.dev[a:b]

    def context(self, page_size: int, max_kv_len: int) -> StepContext:
        """The context the launches are recorded with: device views of the fixed buffers; on the
        host side only what holds for every replay (one token per row, an upper bound of the
        context lengths, no slot ids)."""
        rb = self.rb
        return StepContext(
            num_tokens=rb, num_requests=rb, positions=self.dev_segment("positions"),
            token_req=self.dev_segment("token_req"), cu_seqlens=self.dev_segment("cu"),
            context_lens=self.dev_segment("ctx"), slot_ids=self.dev_segment("slots"),
            block_tables=[self.dev_segment(f"table{g}").view(rb, self.widths[g]) for g in range(self.n_groups)],
            slot_mappings=[self.dev_segment(f"slot_mapping{g}") for g in range(self.n_groups)],
            page_size=page_size, q_lens_host=[1] * rb, context_lens_host=[max_kv_len - 1] * rb,
            slot_ids_host=None, max_q_len=1, max_kv_len=max_kv_len, captured=True,
        )


class EngineCore:
    def __init__(self, model: DecoderModel, config: EngineConfig, num_pages=None):
        """``num_pages`` overrides the configuration's usable pages per cache group."""
        if model.dtype != TORCH_DTYPES[config.dtype]:
            raise ValueError(f"model is bound in {model.dtype}, the engine is configured for {config.dtype}")
        self.model, self.config = model, config
        self.device = model.device
        self.dtype = model.dtype
        self.page_size = config.page_size
        self.plan = model.memory_plan()
        self.group_keys = group_keys_of(self.plan)
        pages = num_pages if num_pages is not None else config.usable_pages
        self.cache = CacheManager(self.group_keys, self.page_size, pages, config.max_num_seqs,
                                  config.enable_prefix_cache, has_state(self.plan))
        self.memories = allocate_memories(self.plan, self.group_keys, pages, self.page_size,
                                          config.max_num_seqs, self.dtype, self.device)
        self.vocab_size = model.spec.vocab_size
        self.kv_bytes_per_token = cache_bytes_per_token(self.plan, self.dtype)
        self._graphs: dict = {}
        self._max_graph_batch = min(config.max_num_seqs, 256)
        # decode steps are recorded and replayed only if every part of the model has declared that
        # it takes the step's values from the device (a part that plans on the host would replay
        # the recorded step's plan for other requests)
        self._replayable = model.replayable()
        self._spare_slot = config.max_num_seqs     # the state row of rows that pad a captured step
        self.graph_replays = 0
        self.steps_followed = 0              # decode steps started before the tokens of the step before were on the host

    # ---- requests
    def start_request(self, request_id, prompt: Optional[Sequence[int]] = None) -> int:
        """Returns the number of prompt tokens found in the prefix cache (0 without a prompt)."""
        return self.cache.start(request_id, prompt)

    def finish_request(self, request_id) -> None:
        self.cache.finish(request_id)

    def has_request(self, request_id) -> bool:
        return self.cache.has(request_id)

    # ---- the step
    def run(self, entries: Sequence[StepEntry], borrow: bool = False) -> torch.Tensor:
        """Float logits [wanted, vocab] in the order of the entries and of their ``want``.
        Raises ``OutOfPages`` before anything ran if a request's tokens have no room.
        ``borrow``: the caller reads the logits before the next call, so a replayed step may
        hand out its own output buffer instead of a copy."""
        entries = [e for e in entries if len(e.tokens) > 0]
        if not entries:
            return torch.empty((0, self.vocab_size), dtype=torch.float32, device=self.device)
        for e in entries:
            for t in e.tokens:
                if not 0 <= int(t) < self.vocab_size:
                    raise ValueError(f"request {e.request_id!r}: token id {t} outside the vocabulary [0, {self.vocab_size})")
            for w in e.want:
                if not 0 <= int(w) < len(e.tokens):
                    raise ValueError(f"request {e.request_id!r}: wanted place {w} outside its {len(e.tokens)} tokens")
        self._reserve_all([(e.request_id, len(e.tokens)) for e in entries])
        self._zero_new_state()
        if self._graphable(entries):
            logits = self._run_decode_graph(entries)
            if not borrow:
                logits = logits.clone()
        else:
            token_ids, ctx, logit_rows = self._build(entries)
            logits = self.model.forward(token_ids, ctx, self.memories, logit_rows)
        for e in entries:
            self.cache.commit(e.request_id, e.tokens)
        return logits

    def _reserve_all(self, needs) -> None:
        """Pages for every (request, new tokens) of a step, or ``OutOfPages`` with no table changed:
        the pools are asked for the sum first, so an entry that does not fit never leaves the
        entries before it with pages they did not have."""
        from ..cache.page_pool import OutOfPages

        cache = self.cache
        promised = [0] * len(self.group_keys)
        for rid, n in needs:
            if not cache.can_store(rid, n, reserve=promised):
                raise OutOfPages(f"request {rid!r}: no pages for {n} more token(s) beside the step's other entries")
            promised = [p + k for p, k in zip(promised, cache.pages_needed(rid, n))]
        for rid, n in needs:
            cache.reserve(rid, n)

    # ---- decode-only steps as replayed HIP graphs
    def _graphable(self, entries) -> bool:
        if not self.config.use_hip_graphs or not self._replayable or len(entries) > self._max_graph_batch:
            return False
        return all(len(e.tokens) == 1 and list(e.want) == [0] for e in entries)

    def _graph_key(self, request_ids, more_tokens: int = 0) -> tuple:
        """(rows, block-table widths) of the captured step that serves these requests, once each of
        them has pages for ``more_tokens`` further tokens."""
        cache = self.cache
        have = [[len(cache.block_table(r, g)) + (cache.pages_needed(r, more_tokens)[g] if more_tokens else 0)
                 for r in request_ids] for g in range(len(self.group_keys))]
        return _batch_bucket(len(request_ids)), tuple(_bucket(max(h), 8) for h in have)

    def follow_decode(self, request_ids: Sequence, token_source: torch.Tensor) -> Optional[torch.Tensor]:
        """One more decode step of exactly these requests (each has one token's logits on the way),
        launched before the tokens are known on the host: row i takes its token from
        ``token_source[i]`` (int32, on the device, written by work already on the stream).  Only a
        step that is already captured and whose pages are free is launched; otherwise None, and
        nothing has changed.  The caller commits each request's token (``commit_decode``) once it
        knows it, before anything else is asked of that request."""
        if not self.config.use_hip_graphs or not self._replayable or not 0 < len(request_ids) <= self._max_graph_batch:
            return None
        cache = self.cache
        g = self._graphs.get(self._graph_key(request_ids, 1))
        if g is None or g.graph is None:
            return None
        from ..cache.page_pool import OutOfPages

        try:
            self._reserve_all([(r, 1) for r in request_ids])
        except OutOfPages:
            return None
        self.steps_followed += 1
        return self._run_decode_graph([StepEntry(r, [0], [0]) for r in request_ids], token_source)

    def commit_decode(self, request_id, token: int) -> None:
        """The token that a step of ``follow_decode`` read for this request from the device."""
        self.cache.commit(request_id, [int(token)])

    def _run_decode_graph(self, entries, token_source: Optional[torch.Tensor] = None) -> torch.Tensor:
        """A step of single tokens, one per request, each wanting its logits: the launch sequence
        is captured once per (batch bucket, table-width bucket) and replayed from fixed buffers;
        rows added to reach the bucket size read the null page and store nothing.  With
        ``token_source`` the tokens are copied from there on the device instead of coming from the
        entries."""
        cache, ps = self.cache, self.page_size
        r = len(entries)
        n_groups = len(self.group_keys)
        key = self._graph_key([e.request_id for e in entries])
        rb, widths = key
        g = self._graphs.get(key)
        if g is None:
            g = self._graphs[key] = _DecodeGraph(rb, widths, n_groups, self.device)
        if g.copied is not None:
            g.copied.synchronize()   # the previous step's upload has left the pinned buffer
        host = g.host
        seg = g.segment
        reqs = [cache.requests[e.request_id] for e in entries]
        ctx_lens = [rc.context_len for rc in reqs]
        for name in ("tokens", "positions", "ctx"):
            seg(host, name)[r:] = 0
        seg(host, "slots")[r:] = self._spare_slot
        seg(host, "tokens")[:r] = [int(e.tokens[0]) for e in entries]
        seg(host, "positions")[:r] = ctx_lens
        seg(host, "ctx")[:r] = ctx_lens
        seg(host, "slots")[:r] = [rc.slot for rc in reqs]
        for gi in range(n_groups):
            sm = seg(host, f"slot_mapping{gi}")
            sm[r:] = -1
            sm[:r] = [rc.tables[gi][c // ps] * ps + c % ps for rc, c in zip(reqs, ctx_lens)]
            # block-table rows are rewritten only when the request in the row or its table changed
            bt = seg(host, f"table{gi}").reshape(rb, widths[gi])
            sig = g.row_signature[gi]
            for i, rc in enumerate(reqs):
                s = (rc.serial, rc.versions[gi])     # the serial, not the id: an id may be used again
                if sig[i] != s:
                    t = rc.tables[gi]
                    bt[i, :len(t)] = t
                    bt[i, len(t):] = 0
                    sig[i] = s
            for i in range(r, rb):
                if sig[i] is not None:
                    bt[i, :] = 0
                    sig[i] = None
        if r < rb:
            # rows that pad the step write the spare state row: it starts from zero in every step, so
            # that a mixer which keeps adding to its state never runs it up to infinity there
            for m in self.memories:
                if m.state is not None:
                    m.state[self._spare_slot].zero_()
        g.dev.copy_(g.host_tensor, non_blocking=True)
        if g.copied is None:
            g.copied = torch.cuda.Event()
        g.copied.record()
        if token_source is not None:
            g.dev_segment("tokens")[:r].copy_(token_source[:r])
        if g.graph is None:
            # first use: run the launches eagerly (this is the step's result), then record them
            ctx = g.context(ps, self.page_size * max(widths, default=1))
            logits = self.model.forward(g.dev_segment("tokens"), ctx, self.memories, g.dev_segment("rows"))
            g.logits = torch.empty_like(logits)
            g.logits.copy_(logits)
            torch.cuda.synchronize()
            graph = torch.cuda.CUDAGraph()
            ctx.extras = {}   # per-step kernel results are recomputed inside the graph; plans stay
            with torch.cuda.graph(graph):
                out = self.model.forward(g.dev_segment("tokens"), ctx, self.memories, g.dev_segment("rows"))
                g.logits.copy_(out)
            g.graph, g.ctx = graph, ctx
        else:
            g.graph.replay()
            self.graph_replays += 1
        return g.logits[:r]

    def _zero_new_state(self) -> None:
        slots = self.cache.take_new_slots()
        if slots and any(m.state is not None for m in self.memories):
            idx = torch.tensor(slots, dtype=torch.long, device=self.device)
            for m in self.memories:
                if m.state is not None:
                    m.state.index_fill_(0, idx, 0)

    def _build(self, entries):
        """All per-token and per-request integers of the step, packed on the host into one
        pinned buffer and copied to the device at once."""
        cache, ps = self.cache, self.page_size
        n_groups = len(self.group_keys)
        q_lens = [len(e.tokens) for e in entries]
        ctx_lens = [cache.context_len(e.request_id) for e in entries]
        slots = [cache.slot(e.request_id) for e in entries]
        n, r = sum(q_lens), len(entries)
        tables = [[cache.block_table(e.request_id, g) for e in entries] for g in range(n_groups)]
        widths = [max(1, max(len(t) for t in tables[g])) for g in range(n_groups)]
        m = sum(len(e.want) for e in entries)

        sizes = [n, n, n, r + 1, r, r, m] + [n] * n_groups + [r * w for w in widths]
        offsets = np.concatenate([[0], np.cumsum(sizes)])
        buf = torch.empty(int(offsets[-1]), dtype=torch.int32, pin_memory=True)
        host = buf.numpy()

        def seg(i):
            return host[offsets[i]:offsets[i + 1]]

        tok, pos, treq, cu, ctxl, slot_ids, rows = (seg(i) for i in range(7))
        cu[0] = 0
        at, row_at = 0, 0
        for i, e in enumerate(entries):
            ql = q_lens[i]
            tok[at:at + ql] = np.asarray(e.tokens, dtype=np.int32)
            pos[at:at + ql] = np.arange(ctx_lens[i], ctx_lens[i] + ql, dtype=np.int32)
            treq[at:at + ql] = i
            for w in e.want:
                rows[row_at] = at + int(w)
                row_at += 1
            at += ql
            cu[i + 1] = at
        ctxl[:] = ctx_lens
        slot_ids[:] = slots
        for g in range(n_groups):
            sm = seg(7 + g)
            at = 0
            for i, e in enumerate(entries):
                sm[at:at + q_lens[i]] = cache.slot_mapping(e.request_id, g, q_lens[i])
                at += q_lens[i]
            bt = seg(7 + n_groups + g).reshape(r, widths[g])
            bt[:] = 0
            for i, t in enumerate(tables[g]):
                bt[i, :len(t)] = t

        dev = buf.to(self.device, non_blocking=True)

        def dseg(i):
            return dev[int(offsets[i]):int(offsets[i + 1])]

        ctx = StepContext(
            num_tokens=n, num_requests=r, positions=dseg(1), token_req=dseg(2), cu_seqlens=dseg(3),
            context_lens=dseg(4), slot_ids=dseg(5),
            block_tables=[dseg(7 + n_groups + g).view(r, widths[g]) for g in range(n_groups)],
            slot_mappings=[dseg(7 + g) for g in range(n_groups)],
            page_size=ps, q_lens_host=q_lens, context_lens_host=ctx_lens, slot_ids_host=slots,
            max_q_len=max(q_lens), max_kv_len=max(c + q for c, q in zip(ctx_lens, q_lens)),
        )
        ctx.extras["pinned"] = buf  # keeps the staging buffer alive until the step has run
        return dseg(0), ctx, dseg(6)
