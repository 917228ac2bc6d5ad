"""Host bookkeeping of one pool of cache pages: reference counts, a free list that is
also the eviction order, and a map from content hashes to pages for prefix reuse.

Reference: ``jllm/engine/paged.py:41-148``.  Same policy: allocation pops the *head* of the
free list (and forgets that page's hash: eviction); release walks a request's pages in
reverse and appends zero-reference pages to the *tail* with hash and contents intact, so
a later ``retain`` can revive them until they are reallocated, and a sequence's last pages
are evicted before its first.  Page 0 is the null page: never allocated, never freed, the
target of table entries that name no page.
"""
from __future__ import annotations

import hashlib
import struct
from typing import Iterable, Optional

NULL_PAGE = 0


class OutOfPages(MemoryError):
    """No free page is left in the pool."""


def chain_hash(parent: bytes, token_ids: Iterable[int]) -> bytes:
    """sha256(parent ‖ tokens as little-endian u32); the root parent is b""
    (``jllm/engine/paged.py:41-46``)."""
    h = hashlib.sha256()
    h.update(parent)
    for t in token_ids:
        h.update(struct.pack("<I", int(t)))
    return h.digest()


class PagePool:
    def __init__(self, num_pages: int):
        """``num_pages`` usable pages with ids 1..num_pages (page 0 is the null page)."""
        if num_pages < 1:
            raise ValueError("a page pool needs at least one usable page")
        self.num_pages = num_pages
        n = num_pages + 1
        self._ref = [0] * n
        self._hash: list = [None] * n
        self._prev = [-1] * n
        self._next = [-1] * n
        self._in_free = [False] * n
        self._head = self._tail = -1
        self._num_free = 0
        self._by_hash: dict = {}
        self.evictions = 0
        for p in range(1, n):
            self._push_tail(p)

    # ---- free list (doubly linked, by page id)
    def _push_tail(self, p: int) -> None:
        self._prev[p], self._next[p] = self._tail, -1
        if self._tail >= 0:
            self._next[self._tail] = p
        else:
            self._head = p
        self._tail = p
        self._in_free[p] = True
        self._num_free += 1

    def _unlink(self, p: int) -> None:
        a, b = self._prev[p], self._next[p]
        if a >= 0:
            self._next[a] = b
        else:
            self._head = b
        if b >= 0:
            self._prev[b] = a
        else:
            self._tail = a
        self._prev[p] = self._next[p] = -1
        self._in_free[p] = False
        self._num_free -= 1

    # ---- public
    @property
    def num_free(self) -> int:
        return self._num_free

    def ref_count(self, page: int) -> int:
        return self._ref[page]

    def page_hash(self, page: int) -> Optional[bytes]:
        return self._hash[page]

    def free_order(self) -> list:
        out, p = [], self._head
        while p >= 0:
            out.append(p)
            p = self._next[p]
        return out

    def allocate(self) -> int:
        """A page with reference count 1; the least recently freed page is taken and, if it
        still carried a hash, that hash is forgotten."""
        p = self._head
        if p < 0:
            raise OutOfPages("no free pages available")
        self._unlink(p)
        if self._hash[p] is not None:
            self._by_hash.pop(self._hash[p], None)
            self._hash[p] = None
            self.evictions += 1
        self._ref[p] = 1
        return p

    def retain(self, page: int) -> None:
        """One more user of a page; a freed page that still holds its contents is revived."""
        if page == NULL_PAGE:
            return
        if self._ref[page] == 0:
            if not self._in_free[page]:
                raise RuntimeError(f"page {page} is neither in use nor free")
            self._unlink(page)
        self._ref[page] += 1

    def release(self, pages: Iterable[int]) -> None:
        """One user less for each page, last page first; pages nobody uses join the tail of the
        free list.  Releasing the null page is a no-op; releasing a free page is an error."""
        for p in reversed(list(pages)):
            if p == NULL_PAGE:
                continue
            if self._ref[p] <= 0:
                raise RuntimeError(f"page {p} released more often than it was taken")
            self._ref[p] -= 1
            if self._ref[p] == 0:
                self._push_tail(p)

    def register_hash(self, page: int, h: bytes) -> None:
        """First writer wins: no-op if the page already has a hash or the hash a page."""
        if page == NULL_PAGE or self._hash[page] is not None or h in self._by_hash:
            return
        self._by_hash[h] = page
        self._hash[page] = h

    def lookup(self, h: bytes) -> Optional[int]:
        return self._by_hash.get(h)

    # ---- self-check used by tests
    def check_invariants(self, held: Optional[dict] = None) -> None:
        """Every usable page is either free (ref 0, on the list once) or in use (ref > 0, off the
        list); hashes and the map agree.  ``held``: page -> number of holders the caller knows of."""
        order = self.free_order()
        assert len(order) == len(set(order)) == self._num_free, "free list broken"
        on_list = set(order)
        for p in range(1, self.num_pages + 1):
            assert (self._ref[p] == 0) == (p in on_list), f"page {p}: ref {self._ref[p]}, on free list {p in on_list}"
            assert self._in_free[p] == (p in on_list)
            if self._hash[p] is not None:
                assert self._by_hash.get(self._hash[p]) == p
            if held is not None:
                assert self._ref[p] == held.get(p, 0), f"page {p}: ref {self._ref[p]}, holders {held.get(p, 0)}"
        assert NULL_PAGE not in on_list and self._ref[NULL_PAGE] == 0
        for h, p in self._by_hash.items():
            assert self._hash[p] == h
