"""The cache manager on the host: the reference's own vectors for the page pool
(tests/test_paged.py of the reference), then invariants under random orders of requests:
no page lost, held twice or freed twice."""
import numpy as np
import pytest

from jax_vllm_amd.cache import CacheManager, OutOfPages, OutOfSlots, PagePool, StateSlotPool, chain_hash


# ---- reference vectors (pool sizes there count the sentinel block: make_manager(8) = 7 usable)
def test_alloc_order_and_reverse_release():
    """tests/test_paged.py:87-106 of the reference."""
    pool = PagePool(7)
    a, b, c = pool.allocate(), pool.allocate(), pool.allocate()
    assert (a, b, c) == (1, 2, 3) and pool.ref_count(a) == 1
    pool.release([a, b, c])
    assert pool.ref_count(a) == 0
    assert pool.free_order() == [4, 5, 6, 7, 3, 2, 1]


def test_null_page_is_never_free():
    """tests/test_paged.py:109-124."""
    pool = PagePool(3)
    assert 0 not in pool.free_order()
    pool.release([0])
    assert 0 not in pool.free_order() and pool.num_free == 3


def test_retain_revives_a_freed_hashed_page():
    """tests/test_paged.py:127-151."""
    pool = PagePool(3)
    b = pool.allocate()
    pool.register_hash(b, b"fake-hash")
    pool.release([b])
    assert pool.ref_count(b) == 0 and pool.page_hash(b) == b"fake-hash"
    pool.retain(b)
    assert pool.ref_count(b) == 1 and b not in pool.free_order()
    pool.retain(b)
    assert pool.ref_count(b) == 2 and b not in pool.free_order()


def test_allocation_evicts_the_hash():
    """tests/test_paged.py:154-172."""
    pool = PagePool(3)
    b = pool.allocate()
    pool.register_hash(b, b"hash-A")
    assert pool.lookup(b"hash-A") == b
    pool.release([b])
    assert [pool.allocate(), pool.allocate(), pool.allocate()] == [2, 3, b]
    assert pool.lookup(b"hash-A") is None and pool.page_hash(b) is None and pool.evictions == 1


def test_duplicate_hash_keeps_the_first_page():
    """tests/test_paged.py:175-185."""
    pool = PagePool(7)
    b1, b2 = pool.allocate(), pool.allocate()
    pool.register_hash(b1, b"hash-X")
    pool.register_hash(b2, b"hash-X")
    assert pool.lookup(b"hash-X") == b1 and pool.page_hash(b1) == b"hash-X" and pool.page_hash(b2) is None


def test_chain_hash():
    """tests/test_paged.py:188-202, and the byte layout of jllm/engine/paged.py:41-46."""
    import hashlib
    import struct

    h0 = chain_hash(b"", [1, 2, 3, 4])
    assert h0 == chain_hash(b"", [1, 2, 3, 4]) != chain_hash(b"", [1, 2, 3, 5])
    assert chain_hash(h0, [5, 6, 7, 8]) != chain_hash(chain_hash(b"", [1, 2, 3, 5]), [5, 6, 7, 8])
    assert h0 == hashlib.sha256(b"".join(struct.pack("<I", t) for t in [1, 2, 3, 4])).digest()


def test_pool_errors():
    pool = PagePool(2)
    a, b = pool.allocate(), pool.allocate()
    with pytest.raises(OutOfPages):
        pool.allocate()
    pool.release([a])
    with pytest.raises(RuntimeError, match="more often"):
        pool.release([a])
    pool.check_invariants({b: 1})


def test_state_slots():
    s = StateSlotPool(3)
    assert [s.acquire(), s.acquire(), s.acquire()] == [0, 1, 2]
    with pytest.raises(OutOfSlots):
        s.acquire()
    s.release(1)
    with pytest.raises(RuntimeError):
        s.release(1)
    assert s.acquire() == 1


# ---- manager
def make(pages=8, page=4, seqs=4, groups=(("full",),), prefix=True):
    return CacheManager(list(groups), page, pages, seqs, prefix)


def test_prefix_reuse_never_covers_the_last_prompt_token():
    m = make(pages=16, page=4)
    prompt = list(range(100, 108))                      # exactly two pages
    assert m.start("a", prompt) == 0
    m.reserve("a", 8)
    m.commit("a", prompt)
    m.finish("a")
    # same prompt again: the first page is taken over, the page of the last token is recomputed
    assert m.start("b", prompt) == 4
    assert m.block_table("b", 0) == [1] and m.context_len("b") == 4
    m.reserve("b", 4)
    assert m.slot_mapping("b", 0, 4) == [p * 4 + o for p in [m.block_table("b", 0)[1]] for o in range(4)]
    m.commit("b", prompt[4:])
    # a longer prompt with the same first two pages takes both (their hashes were registered by a and b)
    assert m.start("c", prompt + [1, 2, 3]) == 8
    # a prompt that differs in the first page takes nothing
    assert m.start("d", [7] + prompt[1:]) == 0
    m.check_invariants()
    assert m.hit_tokens == 12


def test_pages_are_shared_while_in_use_and_hashed_as_they_fill():
    m = make(pages=8, page=4)
    m.start("a", None)
    m.reserve("a", 6)
    m.commit("a", [1, 2, 3, 4, 5, 6])                   # one full page hashed, one partial
    assert m.start("b", [1, 2, 3, 4, 9]) == 4           # shares a's first page while a is running
    page = m.block_table("a", 0)[0]
    assert m.block_table("b", 0) == [page] and m.groups[0].pool.ref_count(page) == 2
    m.finish("a")
    assert m.groups[0].pool.ref_count(page) == 1
    m.reserve("a2" if False else "b", 1)
    m.commit("b", [9])
    m.finish("b")
    m.check_invariants()
    assert m.num_free_pages() == 8


def test_reserve_is_all_or_nothing():
    m = make(pages=3, page=4)
    m.start("a", None)
    m.reserve("a", 8)
    m.start("b", None)
    with pytest.raises(OutOfPages):
        m.reserve("b", 8)
    assert m.block_table("b", 0) == [] and m.num_free_pages() == 1
    assert m.can_store("b", 4) and not m.can_store("b", 5)
    assert m.can_store("b", 4, reserve=[0]) and not m.can_store("b", 4, reserve=[1])
    m.check_invariants()


def test_window_group_gives_back_pages_the_window_has_passed():
    m = make(pages=8, page=4, groups=(("full",), ("window", 6)), prefix=True)
    assert not m.prefix_cache                            # reuse is off when a group is not "full"
    m.start("a", None)
    for step in range(5):
        m.reserve("a", 4)
        m.commit("a", [step] * 4)
    # context 20, window 6: the next query (position 20) reads keys 15..20 -> pages 0..2 are dead
    assert m.block_table("a", 1)[:3] == [0, 0, 0] and all(p > 0 for p in m.block_table("a", 1)[3:])
    assert all(p > 0 for p in m.block_table("a", 0))     # the full group keeps everything
    assert m.num_free_pages(1) == 8 - 2 and m.num_free_pages(0) == 8 - 5
    m.check_invariants()
    m.finish("a")
    m.check_invariants()
    assert m.num_free_pages(0) == m.num_free_pages(1) == 8


@pytest.mark.parametrize("seed", range(6))
def test_random_orders_keep_every_page_accounted_for(seed):
    rng = np.random.default_rng(seed)
    groups = [("full",)] if seed % 2 == 0 else [("full",), ("window", 9)]
    m = CacheManager(groups, 4, 24, 5, enable_prefix_cache=True)
    prompts = [rng.integers(0, 3, size=int(rng.integers(1, 30))).tolist() for _ in range(40)]  # tiny vocabulary: many shared prefixes
    live, fed, nxt = {}, {}, 0
    for _ in range(600):
        action = rng.integers(0, 4)
        if action == 0 and nxt < len(prompts) and m.slots.num_free > 0:
            rid = f"r{nxt}"
            cached = m.start(rid, prompts[nxt])
            assert cached % 4 == 0 and cached < len(prompts[nxt])
            live[rid], fed[rid] = prompts[nxt] + rng.integers(0, 3, size=12).tolist(), cached
            nxt += 1
        elif action in (1, 2) and live:
            rid = list(live)[int(rng.integers(len(live)))]
            n = int(min(rng.integers(1, 9), len(live[rid]) - fed[rid]))
            if n > 0 and m.can_store(rid, n):
                m.reserve(rid, n)
                slots = m.slot_mapping(rid, 0, n)
                assert len(set(slots)) == n
                m.commit(rid, live[rid][fed[rid]:fed[rid] + n])
                fed[rid] += n
                assert m.context_len(rid) == fed[rid]
            elif n > 0:
                with pytest.raises(OutOfPages):
                    m.reserve(rid, n)
        elif action == 3 and live:
            rid = list(live)[int(rng.integers(len(live)))]
            m.finish(rid)
            del live[rid], fed[rid]
        m.check_invariants()
        # no slot of the cache is held by two live requests unless the page is a shared full prefix page
        owners = {}
        for rid in live:
            for idx, p in enumerate(m.block_table(rid, 0)):
                owners.setdefault(p, []).append((rid, idx))
        for p, who in owners.items():
            if len(who) > 1:
                assert len({i for _, i in who}) == 1 and m.groups[0].pool.page_hash(p) is not None
    for rid in list(live):
        m.finish(rid)
    m.check_invariants()
    assert all(g.pool.num_free == 24 for g in m.groups) and m.slots.num_free == 5


def test_table_signature_tells_a_restarted_id_from_its_earlier_life():
    """A copy of a block table is valid as long as the table's signature is unchanged.  The
    signature changes with every change of the table and differs between two starts of the
    same request id, also when both lives made the same number of changes."""
    m = CacheManager([("full",), ("window", 8)], 4, 12, 3, enable_prefix_cache=False)
    seen = set()
    for life in range(3):
        m.start("r")
        m.reserve("r", 8)                  # two pages at once: one change
        sig = m.table_signature("r", 0)
        assert sig not in seen
        seen.add(sig)
        assert m.table_signature("r", 0) == sig            # asking changes nothing
        m.commit("r", list(range(8)))
        assert m.table_signature("r", 0) == sig            # the full group's table did not change
        m.reserve("r", 1)
        assert m.table_signature("r", 0) != sig
        m.commit("r", [1])
        w = m.table_signature("r", 1)
        m.reserve("r", 3)
        m.commit("r", [1, 2, 3])           # position 12 next: the window group gives its first page back
        assert m.block_table("r", 1)[0] == 0 and m.table_signature("r", 1) != w
        m.finish("r")
    # two requests never share a signature either
    m.start("a"), m.start("b")
    m.reserve("a", 4), m.reserve("b", 4)
    assert m.table_signature("a", 0) != m.table_signature("b", 0)
