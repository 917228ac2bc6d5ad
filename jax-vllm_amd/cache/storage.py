"""Device side of the cache: page storage for every run that keeps keys and values, state
rows for every run that keeps state, and the grouping of runs by need.

Every tensor a mixer declares in its ``PagedCacheSpec`` gets ``[pages + 1, *page_shape]`` in
its own type (the engine's by default), zeroed once (page 0, the null page, stays zero and is
never written).  Zero-init follows ``jllm/engine/paged.py:26-38``; the layouts are the mixers'
own (attention: ``parts.spec.kv_cache_spec``).  Nothing here knows what the tensors hold.
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
                for t in p.cache.tensors:
                    kind = dtype if t.dtype is None else _STATE_DTYPES[t.dtype]
                    mem.pages[t.name] = torch.zeros((num_pages[g] + 1, *t.page_shape(page_size)), dtype=kind, device=device)
                mem.group, mem.writes = g, True
            else:
                owner = memories[p.cache_of]
                if not owner.pages:
                    raise ValueError(f"run {p.run} reads the cache of run {p.cache_of}, which keeps none")
                own, other = p.cache, plan[p.cache_of].cache
                if own.tensors != other.tensors:
                    raise ValueError(f"run {p.run} cannot read run {p.cache_of}'s cache: they declare different tensors "
                                     f"({[(t.name, t.token_shape) for t in own.tensors]} against "
                                     f"{[(t.name, t.token_shape) for t in other.tensors]})")
                if other.window is not None and (own.window is None or own.window > other.window):
                    raise ValueError(
                        f"run {p.run} cannot read run {p.cache_of}'s cache: it needs keys that the owner's "
                        f"window of {other.window} has already given back")
                mem.pages, mem.group, mem.writes = owner.pages, owner.group, False
        if p.state is not None:
            # one row per slot and a spare one that belongs to no request
            mem.state = torch.zeros((max_num_seqs + 1, *p.state.shape), dtype=_STATE_DTYPES[p.state.dtype], device=device)
        memories.append(mem)
    return memories


def cache_bytes_per_token(plan, dtype) -> int:
    def item(t):
        return torch.empty((), dtype=dtype if t.dtype is None else _STATE_DTYPES[t.dtype]).element_size()

    return sum(t.elements_per_token * item(t) for p in plan if p.cache and p.cache_of is None for t in p.cache.tensors)
