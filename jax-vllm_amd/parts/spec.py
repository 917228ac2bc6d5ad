"""The vocabulary that parts, models, cache and engine share.

A *part* is one of: token mixer, feed-forward, norm, position encoding, block
arrangement, embedding, head.  A part is constructed from its sizes and constants
alone (it never sees a model configuration), declares the tensors it needs under
local names, and is looked up by ``(category, kind)`` in one registry, so a model
is a list of ``LayerSpec`` chosen layer by layer plus the order they run in.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Callable, Mapping, Optional, Sequence

import torch

# --------------------------------------------------------------------------- tensors of a part


@dataclass(frozen=True)
class TensorSpec:
    """One tensor a part loads.

    role:  "matrix"  – a floating tensor used in the compute type (bfloat16 or float32);
           "vector"  – a small floating tensor always held in float32 (norm weights and the like:
                        a checkpoint's 32-bit values stay 32-bit, 16-bit values widen exactly);
           "table"   – an integer table, held as int32.
    init:  how the random-weights mode fills it: "normal" N(0, std), "norm" 1 + N(0, norm_std),
           "zeros", or "index" (0, 1, 2, ... for integer tables).
    """

    shape: tuple
    role: str = "matrix"
    init: str = "normal"


# --------------------------------------------------------------------------- what a layer keeps per request


@dataclass(frozen=True)
class PagedTensorSpec:
    """One tensor that a mixer keeps per cached token, in pages.

    ``token_shape`` is what one token stores (e.g. ``(kv_heads, head_dim)``).  A page holds
    ``page_size`` tokens; ``slot_axis`` says where the axis of the tokens of a page is put among
    the token's own axes: 0 gives pages ``[page_size, *token_shape]``, ``len(token_shape)`` puts
    it last (a page's tokens are then contiguous per element).  The storage is
    ``[pages + 1, *page_shape]`` with page 0 the null page.  ``dtype`` None: the engine's compute
    type; otherwise "float32", "bfloat16" or "int32".
    """

    name: str
    token_shape: tuple
    slot_axis: int = 0
    dtype: Optional[str] = None

    def __post_init__(self):
        if not 0 <= self.slot_axis <= len(self.token_shape):
            raise ValueError(f"cache tensor {self.name!r}: slot axis {self.slot_axis} outside 0..{len(self.token_shape)}")

    def page_shape(self, page_size: int) -> tuple:
        shape = list(self.token_shape)
        shape.insert(self.slot_axis, int(page_size))
        return tuple(shape)

    @property
    def elements_per_token(self) -> int:
        n = 1
        for s in self.token_shape:
            n *= int(s)
        return n


@dataclass(frozen=True)
class PagedCacheSpec:
    """What a mixer keeps per token in pages: the tensors it declares (a page of each for every
    page id) and which earlier tokens it reads.  ``window`` None: every earlier token is read
    ("full"); otherwise only the last ``window`` are, and older pages are given back.  Mixers with
    the same need share a page pool and a block table (a *group*), whatever tensors they keep."""

    tensors: tuple
    window: Optional[int] = None

    def __post_init__(self):
        names = [t.name for t in self.tensors]
        if len(set(names)) != len(names) or not names:
            raise ValueError(f"a paged cache needs tensors with distinct names, got {names}")

    @property
    def group_key(self) -> tuple:
        return ("window", self.window) if self.window else ("full",)


def kv_cache_spec(num_kv_heads: int, head_dim: int, window: Optional[int] = None) -> PagedCacheSpec:
    """Keys and values of grouped-query attention in the layout its kernels read: a key page is
    ``[kv_heads, page_size, head_dim]`` (one head's keys of a page are contiguous), a value page
    is transposed, ``[kv_heads, head_dim, page_size]`` (8 consecutive keys of one head element are
    16 aligned bytes)."""
    shape = (int(num_kv_heads), int(head_dim))
    return PagedCacheSpec((PagedTensorSpec("k", shape, slot_axis=1), PagedTensorSpec("v", shape, slot_axis=2)), window)


@dataclass(frozen=True)
class StateSpec:
    """State of fixed size per request (one row per slot), zeroed when a request starts."""

    shape: tuple
    dtype: str = "float32"


@dataclass
class LayerMemory:
    """What the cache manager hands one layer run.

    ``pages``: the storage of every tensor the run's mixer declared in its ``PagedCacheSpec``, by
    name, each ``[pages + 1, *page_shape]`` (empty for a mixer without a paged cache);
    ``group`` says which block table / slot mapping of the step applies; ``writes`` is False for
    a run that reads another run's cache.  ``state`` is [slots + 1, *shape] or None; its last row
    belongs to no request (rows that pad a captured step point there).
    """

    pages: dict = field(default_factory=dict)
    group: int = 0
    writes: bool = True
    state: Optional[torch.Tensor] = None


@dataclass
class StepContext:
    """Everything position- and request-indexed that one step's layers may need.

    Tokens of all requests are flattened, request after request.  Device tensors are
    int32.  Host mirrors are Python lists for parts that plan work on the host.

    ``captured``: the launches of this step are recorded once and replayed for later steps
    with other requests in the same rows.  Then only the device tensors carry the step's
    values: ``q_lens_host`` is exact (ones), ``context_lens_host`` holds an upper bound for
    every row, ``slot_ids_host`` is None, and rows that pad the batch have the null page in
    their tables, slot mapping -1 and the spare state slot (the last row of ``LayerMemory.state``).
    Only models whose parts all declare ``replayable = True`` are ever run this way.
    """

    num_tokens: int
    num_requests: int
    positions: torch.Tensor            # [N] absolute position of each token in its request
    token_req: torch.Tensor            # [N] index of the token's request in this step
    cu_seqlens: torch.Tensor           # [R+1] token offsets of the requests
    context_lens: torch.Tensor         # [R] tokens of the request already in the cache before this step
    slot_ids: torch.Tensor             # [R] state slot of each request
    block_tables: list                 # per cache group: [R, max_pages] page ids (0 = no page)
    slot_mappings: list                # per cache group: [N] page * page_size + offset (-1: do not store)
    page_size: int
    q_lens_host: list                  # [R] tokens of each request in this step
    context_lens_host: list            # [R]
    slot_ids_host: Optional[list]      # [R]; None in a captured step
    max_q_len: int = 1
    max_kv_len: int = 1
    extras: dict = field(default_factory=dict)   # per-step results of kernels, shared by parts of one kind
    plans: dict = field(default_factory=dict)    # per-step work lists built on the host and uploaded
    captured: bool = False

    @property
    def decode_only(self) -> bool:
        return self.max_q_len == 1


def is_replayable(part) -> bool:
    """Whether a part's ``forward`` may be recorded once and replayed for later steps: it reads
    the step's values (positions, lengths, tables, slots) from the context's device tensors only
    and uses the host mirrors at most as upper bounds for planning.  A part says so with a class
    or instance attribute ``replayable = True``; a part that says nothing is taken to plan on the
    host and its model's decode steps are never captured."""
    return bool(getattr(part, "replayable", False))


# --------------------------------------------------------------------------- registry of parts

CATEGORIES = ("mixer", "feed_forward", "norm", "position", "block", "embedding", "head")
_PARTS: dict[tuple, Callable[..., Any]] = {}


def register_part(category: str, kind: str, factory: Callable[..., Any]) -> None:
    """Make ``PartSpec(kind, params)`` of this category buildable.  ``factory(**params)``
    returns the part.  Registering an existing name replaces it."""
    if category not in CATEGORIES:
        raise ValueError(f"unknown part category {category!r}; one of {CATEGORIES}")
    _PARTS[(category, kind)] = factory


@dataclass(frozen=True)
class PartSpec:
    kind: str
    params: Mapping[str, Any] = field(default_factory=dict)


def build_part(category: str, spec: PartSpec):
    try:
        factory = _PARTS[(category, spec.kind)]
    except KeyError:
        known = sorted(k for c, k in _PARTS if c == category)
        raise ValueError(f"no {category} part named {spec.kind!r}; registered: {known}") from None
    return factory(**dict(spec.params))


# --------------------------------------------------------------------------- a model as data


@dataclass(frozen=True)
class LayerSpec:
    """One layer: its parts and the prefix of its tensors in the checkpoint."""

    prefix: str                    # e.g. "model.layers.3."
    mixer: PartSpec
    feed_forward: PartSpec
    block: PartSpec
    mixer_prefix: str = ""         # below ``prefix``, e.g. "self_attn."
    feed_forward_prefix: str = ""  # below ``prefix``, e.g. "mlp."
    # local tensor name -> name below ``prefix`` where the checkpoint's differs from the part's
    rename: Mapping[str, str] = field(default_factory=dict)


@dataclass(frozen=True)
class LayerRun:
    """One entry of the execution order.  ``layer`` indexes ``ModelSpec.layers`` (a layer may
    be named by several runs: its weights are shared).  ``cache_of`` None: the run keeps a
    cache and state of its own; otherwise the index of an *earlier run* whose cache it reads
    without writing."""

    layer: int
    cache_of: Optional[int] = None


@dataclass(frozen=True)
class ModelSpec:
    vocab_size: int
    hidden_size: int
    embedding: PartSpec
    embedding_prefix: str
    final_norm: PartSpec
    final_norm_prefix: str
    head: PartSpec
    head_prefix: str
    layers: Sequence[LayerSpec]
    schedule: Sequence[LayerRun]
    tie_head_to_embedding: bool = False

    def __post_init__(self):
        for i, run in enumerate(self.schedule):
            if not 0 <= run.layer < len(self.layers):
                raise ValueError(f"schedule entry {i} names layer {run.layer}, the model has {len(self.layers)}")
            if run.cache_of is not None:
                if not 0 <= run.cache_of < i:
                    raise ValueError(f"schedule entry {i} reads the cache of run {run.cache_of}, which is not earlier")
                if self.schedule[run.cache_of].cache_of is not None:
                    raise ValueError(f"schedule entry {i} reads run {run.cache_of}, which has no cache of its own")
