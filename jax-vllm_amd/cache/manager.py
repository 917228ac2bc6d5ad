"""The cache manager: for every request a block table per cache group, a state slot, the
count of tokens whose keys and values are stored, and the rules by which pages are taken,
shared, and given back.

Layers whose mixers have the same need (all earlier keys; or a window of a given length)
form a *group*: one page pool and one block table per request serve all layers of the
group, each layer having page storage of its own.  Pages of a window group are given back
as soon as the window has passed them; all pages and the slot are given back when the
request ends.  Full pages of the all-keys group are hashed by content (chained over the
prefix) so that a later request with the same prefix takes them instead of recomputing.

Reference: ``jllm/engine/cache.py`` (prefix walk, registration), ``jllm/engine/engine.py:282-314``
(what admission does with hits), ``jllm/engine/paged.py`` (pool).  Differences: a request's
last prompt token is always computed, so a hit never covers the whole prompt and nothing is
ever written into a shared page (the reference re-writes the last cached slot,
``engine.py:309-313``); groups and windows do not exist there.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Optional, Sequence

from .page_pool import NULL_PAGE, OutOfPages, PagePool, chain_hash
from .state_slots import StateSlotPool


@dataclass
class CacheGroup:
    key: tuple                 # ("full",) or ("window", W)
    runs: list                 # schedule entries whose own cache lives in this group
    pool: PagePool

    @property
    def window(self) -> Optional[int]:
        return self.key[1] if self.key[0] == "window" else None


@dataclass
class RequestCache:
    request_id: object
    slot: int
    tokens: list = field(default_factory=list)     # tokens whose keys/values are stored (positions 0..len-1)
    tables: list = field(default_factory=list)     # per group: page id per page index (NULL_PAGE once released)
    hashes: list = field(default_factory=list)     # chain hashes of the full pages hashed so far (full group)
    num_cached_tokens: int = 0                     # tokens taken over from the prefix cache at start
    versions: list = field(default_factory=list)   # per group: bumped whenever the table changes
    serial: int = 0                                # unique per start: a request id used again gets a new one

    @property
    def context_len(self) -> int:
        return len(self.tokens)


class CacheManager:
    def __init__(self, group_keys: Sequence[tuple], page_size: int, num_pages, max_num_seqs: int,
                 enable_prefix_cache: bool = True, has_state: bool = False):
        """``group_keys``: the distinct cache needs in the model, e.g. [("full",), ("window", 128)].
        ``num_pages``: usable pages per group (an int for all, or one per group)."""
        self.page_size = int(page_size)
        if isinstance(num_pages, int):
            num_pages = [num_pages] * len(group_keys)
        self.groups = [CacheGroup(tuple(k), [], PagePool(n)) for k, n in zip(group_keys, num_pages)]
        self.slots = StateSlotPool(max_num_seqs)
        self.requests: dict = {}
        only_full = all(g.key == ("full",) for g in self.groups)
        self.prefix_cache = bool(enable_prefix_cache and only_full and not has_state and self.groups)
        self.hit_tokens = 0
        self.new_slots: list = []   # slots assigned since the engine last zeroed state rows
        self._starts = 0            # requests started so far (the next one's serial)

    # ---- queries
    def has(self, request_id) -> bool:
        return request_id in self.requests

    def context_len(self, request_id) -> int:
        return self.requests[request_id].context_len

    def num_free_pages(self, group: int = 0) -> int:
        return self.groups[group].pool.num_free

    def _pages_for(self, n_tokens: int) -> int:
        return -(-n_tokens // self.page_size)

    def pages_needed(self, request_id, num_new_tokens: int, context_len: Optional[int] = None) -> list:
        """New pages each group must supply so that ``num_new_tokens`` more tokens can be stored.
        For a request that has not started, pass ``request_id=None`` and its ``context_len``."""
        if request_id is not None and request_id in self.requests:
            rc = self.requests[request_id]
            have = [len(t) for t in rc.tables]
            ctx = rc.context_len
        else:
            have = [self._pages_for(context_len or 0)] * len(self.groups)
            ctx = context_len or 0
        need = self._pages_for(ctx + num_new_tokens)
        return [max(0, need - h) for h in have]

    def can_store(self, request_id, num_new_tokens: int, context_len: Optional[int] = None,
                  reserve: Optional[list] = None) -> bool:
        """Whether every group has the free pages for it (``reserve``: pages per group already
        promised to other requests of the step being built)."""
        need = self.pages_needed(request_id, num_new_tokens, context_len)
        reserve = reserve or [0] * len(self.groups)
        return all(g.pool.num_free - r >= n for g, n, r in zip(self.groups, need, reserve))

    # ---- life of a request
    def start(self, request_id, prompt: Optional[Sequence[int]] = None) -> int:
        """Give the request a slot and empty tables; with the prefix cache on and a prompt given,
        take over the longest chain of cached full pages, but never the page of the last prompt
        token.  Returns the number of tokens taken over (a multiple of the page size)."""
        if request_id in self.requests:
            raise KeyError(f"request {request_id!r} already started")
        rc = RequestCache(request_id, self.slots.acquire(), tables=[[] for _ in self.groups],
                          versions=[0] * len(self.groups), serial=self._starts)
        self._starts += 1
        self.new_slots.append(rc.slot)
        self.requests[request_id] = rc
        if self.prefix_cache and prompt is not None and len(prompt) > 1:
            pool = self.groups[0].pool
            parent = b""
            limit = (len(prompt) - 1) // self.page_size
            for i in range(limit):
                h = chain_hash(parent, prompt[i * self.page_size:(i + 1) * self.page_size])
                page = pool.lookup(h)
                if page is None:
                    break
                pool.retain(page)
                rc.tables[0].append(page)
                rc.hashes.append(h)
                parent = h
            n = len(rc.tables[0]) * self.page_size
            rc.tokens = list(prompt[:n])
            rc.num_cached_tokens = n
            self.hit_tokens += n
        return rc.num_cached_tokens

    def reserve(self, request_id, num_new_tokens: int) -> None:
        """Extend the request's tables so that positions context_len .. context_len+n-1 have
        pages.  Raises ``OutOfPages`` (leaving the tables as they were) if a pool runs dry."""
        rc = self.requests[request_id]
        need = self.pages_needed(request_id, num_new_tokens)
        for g, n in zip(self.groups, need):
            if g.pool.num_free < n:
                raise OutOfPages(f"group {g.key}: {n} pages needed, {g.pool.num_free} free")
        for gi, (g, table, n) in enumerate(zip(self.groups, rc.tables, need)):
            for _ in range(n):
                table.append(g.pool.allocate())
            if n:
                rc.versions[gi] += 1

    def slot_mapping(self, request_id, group: int, num_new_tokens: int) -> list:
        """Flat cache slot (page * page_size + offset) of each of the next tokens."""
        rc = self.requests[request_id]
        table, ps, ctx = rc.tables[group], self.page_size, rc.context_len
        out = []
        for pos in range(ctx, ctx + num_new_tokens):
            page = table[pos // ps]
            if page == NULL_PAGE:
                raise RuntimeError(f"request {request_id!r}: position {pos} has no page")
            out.append(page * ps + pos % ps)
        return out

    def block_table(self, request_id, group: int) -> list:
        return self.requests[request_id].tables[group]

    def table_signature(self, request_id, group: int) -> tuple:
        """Equal for two moments only if the block table of this group is the same one with the
        same content: (serial of the start, version of the table).  A request id that is finished
        and started again has another serial, so a copy of its old table is never taken for the
        new one."""
        rc = self.requests[request_id]
        return (rc.serial, rc.versions[group])

    def slot(self, request_id) -> int:
        return self.requests[request_id].slot

    def commit(self, request_id, token_ids: Sequence[int]) -> None:
        """The step has stored keys and values of these tokens: advance the context, hash the
        pages that became full, give back window pages that no later token will read."""
        rc = self.requests[request_id]
        rc.tokens.extend(int(t) for t in token_ids)
        ps, ctx = self.page_size, rc.context_len
        if self.prefix_cache:
            pool, table = self.groups[0].pool, rc.tables[0]
            while (len(rc.hashes) + 1) * ps <= ctx:
                i = len(rc.hashes)
                h = chain_hash(rc.hashes[-1] if rc.hashes else b"", rc.tokens[i * ps:(i + 1) * ps])
                pool.register_hash(table[i], h)
                rc.hashes.append(h)
        for gi, (g, table) in enumerate(zip(self.groups, rc.tables)):
            w = g.window
            if w is None:
                continue
            # the next query sits at position ctx and reads keys > ctx - w: pages that end at or
            # before ctx - w + 1 are dead
            dead_pages = max(0, ctx - w + 1) // ps
            gone = [i for i in range(min(dead_pages, len(table))) if table[i] != NULL_PAGE]
            g.pool.release([table[i] for i in gone])
            for i in gone:
                table[i] = NULL_PAGE
            if gone:
                rc.versions[gi] += 1

    def finish(self, request_id) -> None:
        """Give back everything the request holds."""
        rc = self.requests.pop(request_id)
        for g, table in zip(self.groups, rc.tables):
            g.pool.release(table)
        self.slots.release(rc.slot)

    def take_new_slots(self) -> list:
        s, self.new_slots = self.new_slots, []
        return s

    # ---- self-check used by tests
    def check_invariants(self) -> None:
        for gi, g in enumerate(self.groups):
            held: dict = {}
            for rc in self.requests.values():
                for p in rc.tables[gi]:
                    if p != NULL_PAGE:
                        held[p] = held.get(p, 0) + 1
            g.pool.check_invariants(held)
        slots = [rc.slot for rc in self.requests.values()]
        assert len(slots) == len(set(slots)), "a slot is held twice"
        assert len(slots) + self.slots.num_free == self.slots.num_slots, "a slot is lost"
