"""Rotary position encoding part.  Reference: ``jllm/model/common.py:51-66``.

``inv_freq[i] = theta ** (-2 i / dim)`` for i < dim/2, angle = position * inv_freq in
float; the pair (i, i + dim/2) of a head vector (half-split pairing, the reference's
``_rotate_half``) turns by its angle.  ``rotary_dim`` (default: the whole head) and
``interleaved`` pairing (2i, 2i+1) are parameters; elements past ``rotary_dim`` pass
through.  Cosines and sines of a step's positions are computed once per step, in float,
and shared by every layer with the same constants; the rotation itself runs inside the
attention-input kernel, which takes that table and this part's flags.
"""
from __future__ import annotations

import torch

from ..ops import kernels as K
from .spec import register_part


class RotaryEncoding:
    replayable = True      # the table is computed on the device from the step's positions

    def __init__(self, head_dim: int, theta: float, rotary_dim: int | None = None, interleaved: bool = False):
        self.head_dim = int(head_dim)
        self.theta = float(theta)
        self.rotary_dim = int(rotary_dim) if rotary_dim is not None else self.head_dim
        self.interleaved = bool(interleaved)
        if self.rotary_dim % 2 or not 0 < self.rotary_dim <= self.head_dim:
            raise ValueError(f"rotary_dim {self.rotary_dim} must be even and at most the head size {self.head_dim}")
        self.inv_freq = None

    def tensors(self) -> dict:
        return {}

    def inverse_frequencies(self) -> torch.Tensor:
        """float32 table of rotary_dim/2 entries, computed as the reference does."""
        d = self.rotary_dim
        return 1.0 / (self.theta ** (torch.arange(0, d, 2, dtype=torch.float32) / d))

    def bind(self, tensors: dict, dtype: torch.dtype, device=None) -> None:
        self.inv_freq = self.inverse_frequencies().to(device or "cuda").contiguous()

    def as_rotation(self):
        """(rotary_dim, interleaved): this encoding is a rotation of q and k by position, which the
        mixer's own kernel applies from ``rotation_table``.  A position part that asks nothing of
        the mixer's kernels answers None."""
        return self.rotary_dim, self.interleaved

    def rotation_table(self, ctx):
        """Float cos/sin table of the step's positions for the attention-input kernel."""
        key = ("rope_table", self.theta, self.rotary_dim)
        table = ctx.extras.get(key)
        if table is None:
            table = ctx.extras[key] = K.rope_table(ctx.positions, self.inv_freq)
        return table


register_part("position", "rotary", RotaryEncoding)
