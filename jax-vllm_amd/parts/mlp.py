"""Gated feed-forward.  Reference: ``jllm/model/common.py:69-76``:
``down( silu(gate(x)) * up(x) )``, no biases (SwiGLU); the gate's activation is a parameter, one
of ``ops.kernels.GATE_ACTIVATIONS``.  gate and up are one matrix product against
one weight whose rows alternate gate row j, up row j, so that a gate value and its up value
come out next to each other: for few rows the activation is that product's epilogue, for
many rows a kernel over adjacent pairs.  The activation runs in float."""
from __future__ import annotations

import torch

from ..ops import kernels as K
from .spec import TensorSpec, register_part


class GatedMLP:
    replayable = True

    def __init__(self, hidden_size: int, intermediate_size: int, activation: str = "silu"):
        if activation not in K.GATE_ACTIVATIONS:
            raise ValueError(f"GatedMLP has kernels for {sorted(K.GATE_ACTIVATIONS)}, not for {activation!r}")
        self.hidden_size, self.intermediate_size = int(hidden_size), int(intermediate_size)
        self.activation = activation
        self.w_gate_up = self.w_down = None

    def tensors(self) -> dict:
        h, i = self.hidden_size, self.intermediate_size
        return {
            "gate_proj.weight": TensorSpec((i, h)),
            "up_proj.weight": TensorSpec((i, h)),
            "down_proj.weight": TensorSpec((h, i)),
        }

    def bind(self, tensors: dict, dtype: torch.dtype) -> None:
        g, u = tensors["gate_proj.weight"], tensors["up_proj.weight"]
        self.w_gate_up = torch.stack([g, u], dim=1).reshape(2 * g.shape[0], g.shape[1]).contiguous()
        self.w_down = tensors["down_proj.weight"]

    def takes_unscaled_rows(self, n_rows: int) -> bool:
        """x goes into the gate/up product and nowhere else: the norm before may leave its scale to that product."""
        return K.linear_takes_unscaled_rows(n_rows, self.w_gate_up, gate_pairs=True)

    def forward(self, x, ctx=None) -> torch.Tensor:
        z = K.linear(x, self.w_gate_up, gate_pairs=self.activation)    # gate and up rows alternate in the fused weight
        return K.linear(z, self.w_down, partial_ok=True)   # the next norm adds the partial products


register_part("feed_forward", "gated_mlp", GatedMLP)
