"""Keys of sampling draws (host-only)."""
from __future__ import annotations

import hashlib


def draw_key(seed: int, request_key: int, index: int) -> int:
    """64-bit key (as a signed int64 value) of the draw of a request's ``index``-th token: it
    depends on (seed, request, index) only, so the draw is the same under any batching, cutting
    or recomputation."""
    d = hashlib.blake2b(f"{seed}:{request_key}:{index}".encode(), digest_size=8).digest()
    v = int.from_bytes(d, "little")
    return v - (1 << 64) if v >= (1 << 63) else v
