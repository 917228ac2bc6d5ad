"""Device side of the cache: page storage for every run that keeps keys and values, state
rows for every run that keeps state, and the grouping of runs by need.

Key pages are ``[pages + 1, kv_heads, page_size, head_dim]``, value pages are stored
transposed, ``[pages + 1, kv_heads, head_dim, page_size]``, in the engine's type, zeroed once
(page 0, the null page, stays zero and is never written).  Zero-init follows
``jllm/engine/paged.py:26-38``; the layout differs: the head axis comes before the slot axis
so that one head's keys of a page are contiguous, and values are transposed so that the
matrix-core kernels read 8 consecutive keys of one head element as 16 aligned bytes.
"""
from __future__ import annotations

import torch

from ..parts.spec import LayerMemory

_STATE_DTYPES = {"float32": torch.float32, "bfloat16": torch.bfloat16, "int32": torch.int32}


def group_keys_of(plan) -> list:
    """Distinct cache needs in schedule order of first appearance."""
    keys = []
    for p in plan:
        if p.cache is not None and p.cache_of is None and p.cache.group_key not in keys:
            keys.append(p.cache.group_key)
    return keys


def has_state(plan) -> bool:
    return any(p.state is not None for p in plan)


def allocate_memories(plan, group_keys, num_pages, page_size: int, max_num_seqs: int, dtype, device) -> list:
    """One ``LayerMemory`` per schedule entry.  ``num_pages``: usable pages per group."""
    if isinstance(num_pages, int):
        num_pages = [num_pages] * len(group_keys)
    memories = []
    for p in plan:
        mem = LayerMemory()
        if p.cache is not None:
            if p.cache_of is None:
                g = group_keys.index(p.cache.group_key)
                n, h, d = num_pages[g] + 1, p.cache.num_kv_heads, p.cache.head_dim
                mem.k_pages = torch.zeros((n, h, page_size, d), dtype=dtype, device=device)
                mem.v_pages = torch.zeros((n, h, d, page_size), dtype=dtype, device=device)
                mem.group, mem.writes = g, True
            else:
                owner = memories[p.cache_of]
                if owner.k_pages is None:
                    raise ValueError(f"run {p.run} reads the cache of run {p.cache_of}, which keeps none")
                own, other = p.cache, plan[p.cache_of].cache
                if (own.num_kv_heads, own.head_dim) != (other.num_kv_heads, other.head_dim):
                    raise ValueError(f"run {p.run} cannot read run {p.cache_of}'s cache: head shapes differ")
                if other.window is not None and (own.window is None or own.window > other.window):
                    raise ValueError(
                        f"run {p.run} cannot read run {p.cache_of}'s cache: it needs keys that the owner's "
                        f"window of {other.window} has already given back")
                mem.k_pages, mem.v_pages, mem.group, mem.writes = owner.k_pages, owner.v_pages, owner.group, False
        if p.state is not None:
            # one row per slot and a spare one that belongs to no request
            mem.state = torch.zeros((max_num_seqs + 1, *p.state.shape), dtype=_STATE_DTYPES[p.state.dtype], device=device)
        memories.append(mem)
    return memories


def cache_bytes_per_token(plan, dtype) -> int:
    item = torch.empty((), dtype=dtype).element_size()
    return sum(2 * p.cache.num_kv_heads * p.cache.head_dim * item for p in plan if p.cache and p.cache_of is None)
