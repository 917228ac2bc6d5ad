"""Grouped-query causal attention over a paged cache: the token mixer of Qwen3.

Reference: ``jllm/model/common.py:114-137`` (projections, head layout, output
projection; the reference's projections have no bias, here ``qkv_bias`` and ``o_bias`` are options of the
part), ``:107-111`` (optional per-head q/k RMSNorm before the rotation),
``:173-214`` (scores, mask, softmax, kv head = q head // group).  The three input
projections are one matrix product against the row-concatenated weight; scores,
mask and softmax are float inside the attention kernels; keys are stored after
norm and rotation, values as projected (``jllm/engine/generate.py:54-59``).
"""
from __future__ import annotations

import math
from typing import Optional

import torch

from ..ops import kernels as K
from .spec import (LayerMemory, PagedCacheSpec, PartSpec, StepContext, TensorSpec, build_part, is_replayable,
                   kv_cache_spec, register_part)


class GroupedQueryAttention:
    def __init__(self, hidden_size: int, num_heads: int, num_kv_heads: int, head_dim: int,
                 qk_norm_eps: Optional[float] = None, position: Optional[PartSpec] = None,
                 window: Optional[int] = None, scale: Optional[float] = None, qkv_bias: bool = False,
                 o_bias: bool = False):
        if num_heads % num_kv_heads:
            raise ValueError(f"{num_heads} q heads are not a multiple of {num_kv_heads} kv heads")
        self.hidden_size, self.nq, self.nkv, self.d = int(hidden_size), int(num_heads), int(num_kv_heads), int(head_dim)
        self.qk_norm_eps = qk_norm_eps
        self.window = int(window) if window else None
        self.scale = float(scale) if scale is not None else 1.0 / math.sqrt(self.d)
        self.position = build_part("position", position) if position is not None else None
        # what the position part asks of this mixer's kernels: a rotation of q and k by position
        # (rotary_dim, interleaved), or nothing (a part that acts elsewhere, or no part at all)
        self.rotation = self.position.as_rotation() if self.position is not None else None
        self.qkv_bias, self.o_bias = bool(qkv_bias), bool(o_bias)
        self.w_qkv = self.w_o = self.q_norm = self.k_norm = self.b_qkv = self.b_o = None

    # ---- declarations
    @property
    def replayable(self) -> bool:
        """The kernels take positions, lengths and tables from the device; the host plan of a
        captured step (how many blocks share a request's keys) is made for the upper bound of
        the context lengths and is right for every shorter one."""
        return self.position is None or is_replayable(self.position)

    def tensors(self) -> dict:
        t = {
            "q_proj.weight": TensorSpec((self.nq * self.d, self.hidden_size)),
            "k_proj.weight": TensorSpec((self.nkv * self.d, self.hidden_size)),
            "v_proj.weight": TensorSpec((self.nkv * self.d, self.hidden_size)),
            "o_proj.weight": TensorSpec((self.hidden_size, self.nq * self.d)),
        }
        if self.qk_norm_eps is not None:
            t["q_norm.weight"] = TensorSpec((self.d,), role="vector", init="norm")
            t["k_norm.weight"] = TensorSpec((self.d,), role="vector", init="norm")
        if self.qkv_bias:
            t["q_proj.bias"] = TensorSpec((self.nq * self.d,), role="vector")
            t["k_proj.bias"] = TensorSpec((self.nkv * self.d,), role="vector")
            t["v_proj.bias"] = TensorSpec((self.nkv * self.d,), role="vector")
        if self.o_bias:
            t["o_proj.bias"] = TensorSpec((self.hidden_size,), role="vector")
        return t

    def cache_spec(self) -> Optional[PagedCacheSpec]:
        return kv_cache_spec(self.nkv, self.d, self.window)

    def state_spec(self):
        return None

    def bind(self, tensors: dict, dtype: torch.dtype) -> None:
        self.dtype = dtype
        self.w_qkv = torch.cat(
            [tensors["q_proj.weight"], tensors["k_proj.weight"], tensors["v_proj.weight"]], dim=0
        ).contiguous()
        self.w_o = tensors["o_proj.weight"]
        if self.qk_norm_eps is not None:
            self.q_norm, self.k_norm = tensors["q_norm.weight"], tensors["k_norm.weight"]
        if self.qkv_bias:
            self.b_qkv = torch.cat([tensors["q_proj.bias"], tensors["k_proj.bias"], tensors["v_proj.bias"]]).contiguous()
        if self.o_bias:
            self.b_o = tensors["o_proj.bias"].contiguous()
        if self.position is not None:
            self.position.bind({}, dtype, self.w_o.device)

    def _qkv_parts_ok(self) -> bool:
        """Whether the kernel behind the qkv product (norm, rotation, page write) adds float partial
        products itself: decided by sizes and the declared rotation alone, so the same answer holds
        when the norm before asks and when the product runs."""
        rotary_dim, interleaved = self.rotation if self.rotation is not None else (0, False)
        return K.rope_takes_parts(self.dtype, self.d, interleaved, rotary_dim, self.rotation is not None)

    def takes_unscaled_rows(self, n_rows: int) -> bool:
        """x goes into the qkv product and nowhere else: the norm before may leave its scale to that product."""
        return K.linear_takes_unscaled_rows(n_rows, self.w_qkv, partial_ok=self._qkv_parts_ok(), partial_max_width=None)

    # ---- one step
    def forward(self, x, ctx: StepContext, mem: LayerMemory) -> torch.Tensor:
        n = x.shape[0]
        rotary_dim, interleaved = self.rotation if self.rotation is not None else (0, False)
        cos_sin = self.position.rotation_table(ctx) if self.rotation is not None else None
        # at few rows the projection may come as float partial products, which the next kernel adds
        qkv = K.linear(x, self.w_qkv, partial_max_width=None,       # the rotation kernel adds parts of any width
                       partial_ok=self._qkv_parts_ok())
        if self.b_qkv is not None:
            K.add_bias(qkv, self.b_qkv)
        parts = None
        if qkv.dim() == 3:
            parts, qkv = qkv, torch.empty(qkv.shape[1:], dtype=x.dtype, device=x.device)
        writes = mem.writes
        K.qk_norm_rope_write(
            qkv, ctx.slot_mappings[mem.group] if writes else None, self.q_norm, self.k_norm,
            self.qk_norm_eps or 0.0, cos_sin, rotary_dim, interleaved,
            mem.pages["k"] if writes else None, mem.pages["v"] if writes else None, ctx.page_size,
            self.nq, self.nkv, self.d, parts=parts,
        )
        out = torch.empty((n, self.nq * self.d), dtype=x.dtype, device=x.device)
        from . import attention_backend

        attention_backend.run(self, out, qkv, ctx, mem)
        y = K.linear(out, self.w_o, partial_ok=True)      # the next norm adds the partial products
        if self.b_o is not None:
            K.add_bias(y, self.b_o)
        return y


register_part("mixer", "gqa_attention", GroupedQueryAttention)
