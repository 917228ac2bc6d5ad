"""RMSNorm part.  Reference: ``jllm/model/common.py:44-48``.

``y = x * rsqrt(mean(x^2, last axis) + eps) * weight`` with the mean square, the
inverse root and both products in float.  (The reference rounds the normalised value
to the activation type before the product with the weight; here it is rounded once,
after the product.)
"""
from __future__ import annotations

import torch

from ..ops import kernels as K
from .spec import TensorSpec, register_part


class RMSNorm:
    replayable = True

    def __init__(self, size: int, eps: float):
        self.size, self.eps = int(size), float(eps)
        self.weight = None

    def tensors(self) -> dict:
        return {"weight": TensorSpec((self.size,), role="vector", init="norm")}

    def bind(self, tensors: dict, dtype: torch.dtype) -> None:
        self.weight = tensors["weight"]
        self.dtype = dtype

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        """Norm over the last axis of an activation tensor (any leading shape)."""
        return K.rmsnorm(x, self.weight, self.eps)

    def add_norm(self, h: torch.Tensor, delta, rows=None) -> torch.Tensor:
        """The residual step fused with the norm: ``h += delta`` in the float residual stream,
        returns ``norm(h)`` in the activation type.  With ``rows`` only those rows are normed
        and ``h`` is left alone."""
        n_out = h.shape[0] if rows is None else rows.numel()
        out = torch.empty((n_out, self.size), dtype=self.dtype, device=h.device)
        K.add_rmsnorm(h, delta, self.weight, out, self.eps, rows)
        return out


register_part("norm", "rmsnorm", RMSNorm)
