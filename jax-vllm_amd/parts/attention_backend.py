"""Chooses and plans the attention kernels of one step.

bfloat16 with a head size and page size the matrix-core kernels are built for: requests with
one token in the step go to the decode kernel (keys shared out to several blocks when few
requests would leave the chip idle), all others to the prefill kernel in groups of 64 (query,
head-in-group) rows; a work item names two groups of one request, heaviest items first: two
neighbours where the kernel gives each group waves of its own (they see the same keys), else,
while all blocks are on the chip at once, a group that sees many keys with one that sees few, so
that all blocks carry the same load.  Everything else
(float32, other head sizes) runs the generic float-math kernel.  The plan depends on the
step's lengths, the heads-per-group ratio and whether the layer has a window, so it is built
once per step and shared by all layers alike.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Optional

import torch

from ..ops import kernels as K

TARGET_BLOCKS = 256          # blocks of the decode kernel that fill the chip: one per compute unit (measured: 8 requests of
                             # 1,060 keys over 8 kv heads take 14.2 us with 4 splits, 16.0 with 8; 16 requests 20.3 with 2)
MIN_KEYS_PER_SPLIT = 128     # one 32-key tile for each of a block's 4 waves
RESIDENT_BLOCKS = 2          # blocks of the prefill kernel that a compute unit holds at once


@dataclass
class MfmaPlan:
    prefill_work: Optional[torch.Tensor]   # int32 [n, 3]
    n_prefill: int
    decode_work: Optional[torch.Tensor]    # int32 [n]; None when the step holds decoded tokens only
    n_decode: int
    num_splits: int
    scratch: Optional[torch.Tensor]


def decode_splits(n_decode: int, blocks_per_request: int, max_kv_len: int) -> int:
    base = max(1, n_decode * blocks_per_request)
    by_fill = -(-TARGET_BLOCKS // base)
    by_len = max(1, max_kv_len // MIN_KEYS_PER_SPLIT)
    return max(1, min(by_fill, by_len))


KEY_TILE = 64                # keys of one tile of the prefill kernel


def prefill_work_items(q_lens, context_lens, g: int, window: int, group_rows: int, groups_per_item: int,
                       balance: bool = True):
    """Work items (request, first row of group 0, first row of group 1 or -1) of the prefill kernel
    for the requests with more than one token, heaviest first.  Rows are (query, head-in-group)
    pairs.  With ``balance`` and no window the i-th lightest group of a request is paired with its
    i-th heaviest: every pair then walks about the same number of (row tile, key tile) products,
    which matters when the items are so few that the heaviest one decides the time.  Otherwise
    neighbours are paired: they share nearly all their keys, so every fragment read feeds both."""
    items = []
    for r, (ql, cl) in enumerate(zip(q_lens, context_lens)):
        if ql <= 1:
            continue
        groups = []
        for m0 in range(0, ql * g, group_rows):
            last_row = min(ql * g, m0 + group_rows) - 1
            end = cl + last_row // g + 1
            begin = max(0, cl + m0 // g - window + 1) if window else 0
            groups.append((-(-end // KEY_TILE) - begin // KEY_TILE, m0))
        if groups_per_item < 2:
            items.extend((t, r, m0, -1) for t, m0 in groups)
        elif window or not balance:
            for i in range(0, len(groups) - 1, 2):
                items.append((groups[i][0] + groups[i + 1][0], r, groups[i][1], groups[i + 1][1]))
            if len(groups) % 2:
                items.append((groups[-1][0], r, groups[-1][1], -1))
        else:
            lo, hi = 0, len(groups) - 1          # groups are in ascending order of keys seen
            while lo < hi:
                items.append((groups[lo][0] + groups[hi][0], r, groups[hi][1], groups[lo][1]))
                lo, hi = lo + 1, hi - 1
            if lo == hi:
                items.append((groups[lo][0], r, groups[lo][1], -1))
    items.sort(key=lambda w: -w[0])
    return [(r, a, b) for _, r, a, b in items]


def pair_up_resident_items(items: list, first_round: int) -> list:
    """For a launch whose blocks are all on the chip at once, two to a compute unit: the ``first_round`` heaviest
    items (the blocks that get a unit to themselves at first) stay in descending order and the others follow in
    ASCENDING order.  The hardware hands out blocks in the order of their numbers and comes back to the first unit
    after one round, so the unit with the heaviest item gets the lightest one beside it (2,048 tokens, 32 q heads
    over 8 kv heads of 128: 53.9 against 58.3 us; with more items than fit at once, heaviest first stays the
    rule: 94.8 against 103.3 us at 3,072)."""
    return items[:first_round] + items[first_round:][::-1]


def prefill_item_shape(rows: int, nkv: int, group_rows: int, kernel_groups: int, compute_units: int,
                       waves_split: bool = False):
    """(groups per work item, whether light groups are paired with heavy ones) for a step with
    ``rows`` (query, head-in-group) rows per kv head in its prompt portions.  A kernel whose groups
    have waves of their own (``waves_split``) always gets neighbouring pairs: half of a block's waves
    would idle through the keys that only one group sees (2,048 tokens, 32 q heads over 8 kv heads
    of 128: 64 against 78 us; one group per item: 88).  For the other kernel, measured on the same
    heads: while items of two groups would not even give every compute unit a block,
    items of one group do better although every block then loads its keys for half the rows
    (512 tokens after 3,000: 111 against 135 us; after 16,000: 507 against 622); balancing wins
    while all blocks are on the chip at once, two per compute unit (2,048 tokens, 512 blocks: 88
    against 98 us); one more block and the equal loads need a whole further round, so neighbours
    that share their keys, heaviest first, win from there (2,304 tokens, 576 blocks: 111 against
    137 us; 8,192: 887 against 1,036)."""
    if waves_split:
        return kernel_groups, False
    blocks = -(-rows // (group_rows * kernel_groups)) * nkv
    if kernel_groups > 1 and blocks <= compute_units:
        return 1, True
    return kernel_groups, blocks <= RESIDENT_BLOCKS * compute_units


def plan_mfma(ctx, nq: int, nkv: int, head_dim: int, window: int, device) -> MfmaPlan:
    g = nq // nkv
    group_rows, kernel_groups = K.attn_prefill_geometry(head_dim)
    rows = sum(ql * g for ql in ctx.q_lens_host if ql > 1)
    groups_per_item, balance = prefill_item_shape(rows, nkv, group_rows, kernel_groups, K.compute_units(device),
                                                  K.attn_prefill_waves_split(head_dim))
    prefill = prefill_work_items(ctx.q_lens_host, ctx.context_lens_host, g, window, group_rows, groups_per_item,
                                 balance=balance)
    cus = K.compute_units(device)
    if cus < len(prefill) * nkv <= RESIDENT_BLOCKS * cus:
        prefill = pair_up_resident_items(prefill, cus // nkv)
    decode = [r for r, ql in enumerate(ctx.q_lens_host) if ql == 1]
    max_kv_decode = max([ctx.context_lens_host[r] + 1 for r in decode], default=1)
    splits = decode_splits(len(decode), nkv * (-(-g // 16)), max_kv_decode) if decode else 1
    if decode:      # a very wide block table is taken split by split
        widest = max(t.shape[1] for t in ctx.block_tables)
        splits = max(splits, K.attn_decode_min_splits(widest, ctx.page_size))
    decode_only = len(decode) == len(ctx.q_lens_host)       # requests 0, 1, ...: the kernel needs no list
    flat = [x for item in prefill for x in item] + ([] if decode_only else decode)
    dev = torch.tensor(flat, dtype=torch.int32).pin_memory().to(device, non_blocking=True) if flat else None
    n_pre = len(prefill)
    scratch = None
    if decode and splits > 1:
        scratch = torch.empty(K.attn_decode_scratch_floats(len(decode), nq, splits, head_dim),
                              dtype=torch.float32, device=device)
    return MfmaPlan(dev[: 3 * n_pre] if n_pre else None, n_pre,
                    dev[3 * n_pre:] if decode and not decode_only else None, len(decode), splits, scratch)


def run(att, out, qkv, ctx, mem) -> None:
    q_row_stride = (att.nq + 2 * att.nkv) * att.d
    if not K.mfma_attention_supported(qkv.dtype, att.d, ctx.page_size):
        K.paged_attention_generic(
            out, qkv, q_row_stride, mem.pages["k"], mem.pages["v"], ctx.block_tables[mem.group], ctx.token_req,
            ctx.positions, att.nq, att.nkv, att.d, att.scale, att.window or 0,
        )
        return
    key = ("mfma_attention_plan", att.nq, att.nkv, att.d, bool(att.window))
    plan = ctx.plans.get(key)
    if plan is None:
        plan = ctx.plans[key] = plan_mfma(ctx, att.nq, att.nkv, att.d, att.window or 0, qkv.device)
    tables = ctx.block_tables[mem.group]
    if plan.n_prefill:
        K.attn_prefill_mfma(out, qkv, q_row_stride, mem.pages["k"], mem.pages["v"], tables, ctx.cu_seqlens,
                            ctx.context_lens, plan.prefill_work, plan.n_prefill, att.nq, att.nkv, att.d, att.scale,
                            att.window or 0)
    if plan.n_decode:
        K.attn_decode_mfma(out, qkv, q_row_stride, mem.pages["k"], mem.pages["v"], tables, ctx.cu_seqlens,
                           ctx.context_lens, plan.decode_work, plan.n_decode, att.nq, att.nkv, att.d, att.scale,
                           att.window or 0, plan.num_splits, plan.scratch)
