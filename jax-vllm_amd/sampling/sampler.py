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


class Sampler:
    def __init__(self, device):
        self.device = device

    def sample(self, logits: torch.Tensor, temperatures: Sequence[float], keys: Sequence[int]) -> list:
        """One token id per row of ``logits`` [M, V] (float32, on the device)."""
        m = logits.shape[0]
        if m == 0:
            return []
        if all(t <= 0.0 for t in temperatures):
            out = K.sample(logits)
        else:
            temp = torch.tensor(list(temperatures), dtype=torch.float32, device=self.device)
            key = torch.tensor(list(keys), dtype=torch.int64, device=self.device)
            out = K.sample(logits, temp, key)
        ids = out.tolist()
        vocab = logits.shape[1]
        bad = [i for i, t in enumerate(ids) if not 0 <= t < vocab]
        if bad:
            # the kernel answers "no token" (the vocabulary size) for a row without any comparable value
            raise FloatingPointError(f"logits row(s) {bad} of {m} hold no finite maximum (NaN): no token can be chosen")
        return ids
