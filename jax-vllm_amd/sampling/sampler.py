"""Token choice above the step function.

Greedy: argmax of the float logits, lowest index on ties (reference:
``jllm/engine/generate.py:142``, ``jllm/engine/state.py:66``; it is the only rule the
reference has).  Temperature: a draw from ``softmax(logits / T)`` computed in float.  The
draw of a request's k-th token depends on (seed, request, k) and that token's logits only,
so it is the same under any batching, cutting or recomputation.
"""
from __future__ import annotations

from typing import Sequence

import torch

from ..ops import kernels as K
from .keys import draw_key  # noqa: F401  (re-exported)


class Drawn:
    """Tokens that the GPU is still choosing: ``tokens`` on the device (int32, one per row), their copy to
    pinned host memory under way, and the event after that copy."""

    def __init__(self, tokens: torch.Tensor, host: torch.Tensor, copied, rows: int, vocab: int):
        self.tokens, self.host, self.copied, self.rows, self.vocab = tokens, host, copied, rows, vocab


class Sampler:
    HOST_BUFFERS = 4          # pinned buffers in turn: more than the steps that are ever under way at once

    def __init__(self, device):
        self.device = device
        self._host, self._turn = [], 0

    def _pinned(self, rows: int) -> dict:
        """The next set of pinned host buffers (token ids back, temperatures and keys out).  A set is
        used again only after ``HOST_BUFFERS`` further launches, and a launch is finished (its event
        awaited) before the launch after the next one starts, so no copy is still reading or
        writing it."""
        if len(self._host) < self.HOST_BUFFERS:
            self._host.append(None)
        self._turn = (self._turn + 1) % len(self._host)
        have = self._host[self._turn]
        if have is None or have["tokens"].numel() < rows:
            n = max(rows, 64)
            have = self._host[self._turn] = {
                "tokens": torch.empty(n, dtype=torch.int32, pin_memory=True),
                "temperature": torch.empty(n, dtype=torch.float32, pin_memory=True),
                "keys": torch.empty(n, dtype=torch.int64, pin_memory=True),
            }
        return have

    def launch(self, logits: torch.Tensor, temperatures: Sequence[float], keys: Sequence[int]) -> Drawn:
        """Start choosing one token id per row of ``logits`` [M, V] (float32, on the device) and copying
        them to the host; nothing here waits for the GPU."""
        m = logits.shape[0]
        host = self._pinned(m)
        if all(t <= 0.0 for t in temperatures):
            out = K.sample(logits)
        else:
            # through pinned memory and without waiting: a copy from pageable memory would hold the host
            # until the logits are there, and the step after this one could not be started ahead
            host["temperature"][:m] = torch.as_tensor(list(temperatures), dtype=torch.float32)
            host["keys"][:m] = torch.as_tensor(list(keys), dtype=torch.int64)
            temp = host["temperature"][:m].to(self.device, non_blocking=True)
            key = host["keys"][:m].to(self.device, non_blocking=True)
            out = K.sample(logits, temp, key)
        host["tokens"][:m].copy_(out, non_blocking=True)
        copied = torch.cuda.Event()
        copied.record()
        return Drawn(out, host["tokens"], copied, m, logits.shape[1])

    def finish(self, drawn: Drawn) -> list:
        """The token ids of a ``launch``, once they are there."""
        drawn.copied.synchronize()
        ids = drawn.host[:drawn.rows].tolist()
        bad = [i for i, t in enumerate(ids) if not 0 <= t < drawn.vocab]
        if bad:
            # the kernel answers "no token" (the vocabulary size) for a row without any comparable value
            raise FloatingPointError(
                f"logits row(s) {bad} of {drawn.rows} hold no finite maximum (NaN): no token can be chosen")
        return ids

    def sample(self, logits: torch.Tensor, temperatures: Sequence[float], keys: Sequence[int]) -> list:
        """One token id per row of ``logits`` [M, V] (float32, on the device)."""
        if logits.shape[0] == 0:
            return []
        return self.finish(self.launch(logits, temperatures, keys))
