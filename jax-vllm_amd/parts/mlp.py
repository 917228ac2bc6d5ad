"""Gated feed-forward (SwiGLU).  Reference: ``jllm/model/common.py:69-76``:
``down( silu(gate(x)) * up(x) )``, no biases.  gate and up are one matrix product
against the row-concatenated weight; the activation runs in float."""
from __future__ import annotations

import torch

from ..ops import kernels as K
from .spec import TensorSpec, register_part


class GatedMLP:
    def __init__(self, hidden_size: int, intermediate_size: int, activation: str = "silu"):
        if activation != "silu":
            raise ValueError(f"GatedMLP has kernels for 'silu' only, not {activation!r}")
        self.hidden_size, self.intermediate_size = int(hidden_size), int(intermediate_size)
        self.w_gate_up = self.w_down = None

    def tensors(self) -> dict:
        h, i = self.hidden_size, self.intermediate_size
        return {
            "gate_proj.weight": TensorSpec((i, h)),
            "up_proj.weight": TensorSpec((i, h)),
            "down_proj.weight": TensorSpec((h, i)),
        }

    def bind(self, tensors: dict, dtype: torch.dtype) -> None:
        self.w_gate_up = torch.cat([tensors["gate_proj.weight"], tensors["up_proj.weight"]], dim=0).contiguous()
        self.w_down = tensors["down_proj.weight"]

    def forward(self, x: torch.Tensor, ctx=None) -> torch.Tensor:
        gate_up = K.linear(x, self.w_gate_up)
        if gate_up.shape[0] <= 2 and K.skinny_applies(gate_up, self.w_down):
            # one or two rows: the activation runs inside the second product's prologue (every
            # block of that product redoes it, which costs more than a kernel beyond two rows)
            return K.gemm_skinny(gate_up, self.w_down, gate_up.dtype, silu_gate_up=True)
        return K.linear(K.silu_mul(gate_up), self.w_down)


register_part("feed_forward", "gated_mlp", GatedMLP)
