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
    may_leave_scale = True     # ``add_norm`` takes ``unscaled_ok`` (a norm part without this attribute is never asked)

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

    def add_norm(self, h: torch.Tensor, delta, rows=None, unscaled_ok: bool = False):
        """The residual step fused with the norm: ``h += delta`` in the float residual stream,
        returns ``norm(h)`` in the activation type.  With ``rows`` only those rows are normed
        and ``h`` is left alone.  With ``unscaled_ok`` the reader multiplies the rows by a matrix
        through ``K.linear`` and nothing else: for the few rows of a decode step whose ``delta``
        comes as partial products the result may then be ``K.UnscaledRows`` (``h * weight`` with
        the scale left to that product's epilogue), whose residual step is shared out to many blocks
        a row."""
        if (unscaled_ok and rows is None and delta is not None and delta.dim() == 3
                and K.unscaled_rows_possible(self.dtype, h.shape[0], self.size)):
            return K.add_parts_unscaled(h, delta, self.weight, self.eps)
        n_out = h.shape[0] if rows is None else rows.numel()
        out = torch.empty((n_out, self.size), dtype=self.dtype, device=h.device)
        K.add_rmsnorm(h, delta, self.weight, out, self.eps, rows)
        return out


register_part("norm", "rmsnorm", RMSNorm)
