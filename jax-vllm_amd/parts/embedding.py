"""Token embedding and output head.  Reference: ``jllm/model/common.py:35-41`` (row gather,
``x @ W.T`` without bias) and ``jllm/model/weights.py:143-146`` (a tied head is the
embedding table itself, one buffer)."""
from __future__ import annotations

import torch

from ..ops import kernels as K
from .spec import TensorSpec, register_part


class TokenEmbedding:
    replayable = True

    def __init__(self, vocab_size: int, hidden_size: int):
        self.vocab_size, self.hidden_size = int(vocab_size), int(hidden_size)
        self.weight = None

    def tensors(self) -> dict:
        return {"weight": TensorSpec((self.vocab_size, self.hidden_size))}

    def bind(self, tensors: dict, dtype: torch.dtype) -> None:
        self.weight = tensors["weight"]

    def forward(self, ids: torch.Tensor, ctx=None) -> torch.Tensor:
        """Float residual stream [tokens, hidden] of the rows ``ids`` (int32; an id outside the table
        gives a row of NaN).  ``ctx`` is the step's ``StepContext`` (positions, token -> request, ...);
        this embedding needs none of it."""
        h = torch.empty((ids.numel(), self.hidden_size), dtype=torch.float32, device=ids.device)
        K.embedding(h, self.weight, ids)
        return h


class LinearHead:
    replayable = True

    def __init__(self, vocab_size: int, hidden_size: int):
        self.vocab_size, self.hidden_size = int(vocab_size), int(hidden_size)
        self.weight = None

    def tensors(self) -> dict:
        return {"weight": TensorSpec((self.vocab_size, self.hidden_size))}

    def bind(self, tensors: dict, dtype: torch.dtype) -> None:
        self.weight = tensors["weight"]

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        """Float logits [rows, vocab]."""
        return K.linear(x, self.weight, out_dtype=torch.float32)


register_part("embedding", "token_embedding", TokenEmbedding)
register_part("head", "linear_head", LinearHead)
