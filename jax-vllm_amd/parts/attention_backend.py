"""Chooses and plans the attention kernels of one step.

bfloat16 with a head size and page size the matrix-core kernels are built for: requests with
one token in the step go to the decode kernel (keys shared out to several blocks when few
requests would leave the chip idle), all others to the prefill kernel in blocks of 128 (or 64)
(query, head-in-group) rows, heaviest blocks first.  Everything else (float32, other head
sizes) runs the generic float-math kernel.  The plan depends on the step's lengths and on
the heads-per-group ratio only, so it is built once per step and shared by all layers.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Optional

import torch

from ..ops import kernels as K

TARGET_BLOCKS = 512          # about two blocks per compute unit
MIN_KEYS_PER_SPLIT = 128     # one 32-key tile for each of a block's 4 waves


@dataclass
class MfmaPlan:
    prefill_work: Optional[torch.Tensor]   # int32 [n, 2]
    n_prefill: int
    decode_work: Optional[torch.Tensor]    # int32 [n]
    n_decode: int
    num_splits: int
    scratch: Optional[torch.Tensor]


def decode_splits(n_decode: int, blocks_per_request: int, max_kv_len: int) -> int:
    base = max(1, n_decode * blocks_per_request)
    by_fill = -(-TARGET_BLOCKS // base)
    by_len = max(1, max_kv_len // MIN_KEYS_PER_SPLIT)
    return max(1, min(by_fill, by_len))


def plan_mfma(ctx, nq: int, nkv: int, head_dim: int, device) -> MfmaPlan:
    g = nq // nkv
    rows_per_block = K.attn_prefill_rows(head_dim)
    prefill, decode = [], []
    max_kv_decode = 1
    for r, (ql, cl) in enumerate(zip(ctx.q_lens_host, ctx.context_lens_host)):
        if ql == 1:
            decode.append(r)
            max_kv_decode = max(max_kv_decode, cl + 1)
        else:
            for m0 in range(0, ql * g, rows_per_block):
                last_row = min(ql * g, m0 + rows_per_block) - 1
                prefill.append((cl + last_row // g + 1, r, m0))
    prefill.sort(key=lambda w: -w[0])
    splits = decode_splits(len(decode), nkv * (-(-g // 16)), max_kv_decode) if decode else 1
    flat = [x for _, r, m0 in prefill for x in (r, m0)] + decode
    dev = torch.tensor(flat, dtype=torch.int32).pin_memory().to(device, non_blocking=True) if flat else None
    n_pre = len(prefill)
    scratch = None
    if decode and splits > 1:
        scratch = torch.empty(K.attn_decode_scratch_floats(len(decode), nq, splits, head_dim),
                              dtype=torch.float32, device=device)
    return MfmaPlan(dev[: 2 * n_pre] if n_pre else None, n_pre, dev[2 * n_pre:] if decode else None, len(decode),
                    splits, scratch)


def run(att, out, qkv, ctx, mem) -> None:
    q_row_stride = (att.nq + 2 * att.nkv) * att.d
    if not K.mfma_attention_supported(qkv.dtype, att.d, ctx.page_size):
        K.paged_attention_generic(
            out, qkv, q_row_stride, mem.k_pages, mem.v_pages, ctx.block_tables[mem.group], ctx.token_req,
            ctx.positions, att.nq, att.nkv, att.d, att.scale, att.window or 0,
        )
        return
    key = ("mfma_attention_plan", att.nq, att.nkv, att.d)
    plan = ctx.plans.get(key)
    if plan is None:
        plan = ctx.plans[key] = plan_mfma(ctx, att.nq, att.nkv, att.d, qkv.device)
    tables = ctx.block_tables[mem.group]
    if plan.n_prefill:
        K.attn_prefill_mfma(out, qkv, q_row_stride, mem.k_pages, mem.v_pages, tables, ctx.cu_seqlens,
                            ctx.context_lens, plan.prefill_work, plan.n_prefill, att.nq, att.nkv, att.d, att.scale,
                            att.window or 0)
    if plan.n_decode:
        K.attn_decode_mfma(out, qkv, q_row_stride, mem.k_pages, mem.v_pages, tables, ctx.cu_seqlens,
                           ctx.context_lens, plan.decode_work, plan.n_decode, att.nq, att.nkv, att.d, att.scale,
                           att.window or 0, plan.num_splits, plan.scratch)
