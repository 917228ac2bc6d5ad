"""Typed engine configuration.

The reference passes these as arguments of ``make_driver`` (``jllm/engine/engine.py:63-94``:
``max_num_seqs``, ``max_model_len``, ``max_prefill_len``, ``block_size``, ``num_blocks``,
``dtype``).  Here the prefill limit per step is a token budget shared by all requests
(``max_num_batched_tokens``), prompts are cut to fit it, and the page pool may be smaller
than the worst case (the scheduler preempts when pages run out).
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Optional

from .errors import ConfigError

DTYPES = {"bf16": "bfloat16", "bfloat16": "bfloat16", "fp32": "float32", "float32": "float32"}


def canonical_dtype(name: str) -> str:
    try:
        return DTYPES[name]
    except KeyError:
        raise ConfigError(f"dtype must be one of {sorted(DTYPES)}, got {name!r}") from None


@dataclass(frozen=True)
class EngineConfig:
    dtype: str = "bfloat16"              # "bf16"/"bfloat16" (serving kernels) or "fp32"/"float32" (true 32-bit path)
    block_size: int = 16                 # tokens per cache page (reference: block_size=16)
    num_blocks: Optional[int] = None     # pages per cache group, the null page included (reference: num_blocks,
                                         # 1 + max_num_seqs * max_model_len / block_size when None)
    max_num_seqs: int = 4                # requests running at once (reference default 4)
    max_model_len: int = 2048            # prompt + generated tokens of one request (reference default 2048)
    max_prefill_len: Optional[int] = None  # longest prompt accepted; None: max_model_len (reference: same)
    max_num_batched_tokens: int = 2048   # token budget of one step (decode tokens + prompt portions)
    max_chunk: Optional[int] = None      # largest prompt portion of one request in one step; None: the budget
    enable_prefix_cache: bool = True     # reuse full pages of equal prompt prefixes
    use_hip_graphs: bool = True          # replay captured decode-only steps
    decode_ahead: bool = True            # start the decode step after a captured one before its tokens reach the host
    tune_library: bool = False           # at prewarm, let the matrix library time its own kernels for the products it is given
                                         # (steps of more than 64 rows) instead of taking its first guess
    seed: int = 0                        # default sampling seed

    def __post_init__(self):
        object.__setattr__(self, "dtype", canonical_dtype(self.dtype))
        for name in ("block_size", "max_num_seqs", "max_model_len", "max_num_batched_tokens"):
            if getattr(self, name) <= 0:
                raise ConfigError(f"{name} must be positive")
        if self.num_blocks is not None and self.num_blocks < 2:
            raise ConfigError("num_blocks must be at least 2 (the null page and one usable page)")
        if self.max_chunk is not None and self.max_chunk <= 0:
            raise ConfigError("max_chunk must be positive")
        if self.max_prefill_len is not None and self.max_prefill_len > self.max_model_len:
            raise ConfigError("max_prefill_len must be <= max_model_len")

    @property
    def page_size(self) -> int:
        return self.block_size

    @property
    def pages_per_request(self) -> int:
        return -(-self.max_model_len // self.block_size)

    @property
    def prompt_limit(self) -> int:
        return self.max_prefill_len if self.max_prefill_len is not None else self.max_model_len

    @property
    def usable_pages(self) -> int:
        """Pages that can hold tokens; the default pool is the worst case the reference insists
        on (``jllm/engine/engine.py:85-88``): every slot at full length."""
        if self.num_blocks is not None:
            return self.num_blocks - 1
        return self.max_num_seqs * self.pages_per_request

    @property
    def chunk_limit(self) -> int:
        return min(self.max_chunk or self.max_num_batched_tokens, self.max_num_batched_tokens)
