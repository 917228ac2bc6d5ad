"""The host-side plan of the prefill attention kernel: which rows go to which block."""
import random

from jax_vllm_amd.parts.attention_backend import (KEY_TILE, decode_splits, pair_up_resident_items, prefill_item_shape,
                                                   prefill_work_items)


def _tiles(cl, m0, ql, g, rows, window):
    last_row = min(ql * g, m0 + rows) - 1
    end = cl + last_row // g + 1
    begin = max(0, cl + m0 // g - window + 1) if window else 0
    return -(-end // KEY_TILE) - begin // KEY_TILE


def test_every_row_is_in_exactly_one_group():
    rng = random.Random(0)
    for _ in range(200):
        g = rng.choice([1, 2, 4, 5, 20])
        window = rng.choice([0, 0, 7, 100])
        per_item = rng.choice([1, 2])
        q_lens = [rng.choice([1, 2, 3, 17, 64, 65, 300]) for _ in range(rng.randint(1, 4))]
        ctx = [rng.choice([0, 1, 63, 64, 1000]) for _ in q_lens]
        items = prefill_work_items(q_lens, ctx, g, window, 64, per_item)
        seen = sorted((r, m0) for r, a, b in items for m0 in (a, b) if m0 >= 0)
        want = sorted((r, m0) for r, ql in enumerate(q_lens) if ql > 1 for m0 in range(0, ql * g, 64))
        assert seen == want
        assert all(a >= 0 for _, a, _ in items)
        if per_item == 1:
            assert all(b == -1 for _, _, b in items)


def test_single_token_requests_are_left_to_the_decode_kernel():
    assert prefill_work_items([1, 1], [5, 9], 4, 0, 64, 2) == []


def test_pairs_balance_the_load_and_heaviest_come_first():
    ql, g = 2048, 4
    items = prefill_work_items([ql], [0], g, 0, 64, 2)
    loads = [sum(_tiles(0, m0, ql, g, 64, 0) for m0 in (a, b) if m0 >= 0) for _, a, b in items]
    assert loads == sorted(loads, reverse=True)
    assert max(loads) - min(loads) <= 1                      # unpaired, the spread would be 31
    assert len(items) == ql * g // 128


def test_window_pairs_neighbours():
    items = prefill_work_items([512], [0], 1, 64, 64, 2)
    assert sorted((a, b) for _, a, b in items) == [(m0, m0 + 64) for m0 in range(0, 512, 128)]
    items = prefill_work_items([512], [0], 1, 0, 64, 2, balance=False)
    assert [(a, b) for _, a, b in items] == [(m0, m0 + 64) for m0 in range(384, -1, -128)]   # heaviest first


def test_items_that_are_all_on_the_chip_at_once_meet_heavy_with_light():
    """Two blocks to a compute unit, handed out in the order of their numbers: item i and item i + n/2 share a
    unit, so the lighter half runs in ascending order and every unit gets the same load."""
    ql, g = 2048, 4
    items = prefill_work_items([ql], [0], g, 0, 64, 2, balance=False)        # neighbours paired: loads 64, 62, ..., 2 tiles
    loads = lambda its: [sum(_tiles(0, m0, ql, g, 64, 0) for m0 in (a, b) if m0 >= 0) for _, a, b in its]
    paired = pair_up_resident_items(items, 256 // 8)                         # 512 blocks on 256 units: 32 items a round
    assert sorted(paired) == sorted(items)
    n = len(items)
    sums = [x + y for x, y in zip(loads(paired)[:n // 2], loads(paired)[n // 2:])]
    assert max(sums) - min(sums) <= 1
    before = [x + y for x, y in zip(loads(items)[:n // 2], loads(items)[n // 2:])]
    assert max(before) - min(before) >= 30
    # 48 items of 8 blocks on 256 units: the 16 of the second round meet the 16 heaviest, lightest with heaviest
    assert pair_up_resident_items(items[:48], 32) == items[:32] + items[32:48][::-1]


def test_decode_splits_fill_the_chip_but_keep_a_tile_per_wave():
    assert decode_splits(1, 8, 100) == 1                     # too few keys to share out
    assert decode_splits(1, 8, 8192) == 32                   # 8 blocks a split: 256 blocks fill the chip
    assert decode_splits(8, 8, 1061) == 4
    assert decode_splits(64, 8, 8192) == 1                   # enough blocks already


def test_item_shape_follows_the_fill_of_the_chip():
    """Few rows: items of one group, so that more blocks than compute units exist at all; more:
    two groups, light paired with heavy; many: two neighbouring groups."""
    shape = lambda tokens: prefill_item_shape(tokens * 4, 8, 64, 2, 256)     # 32 q heads over 8 kv heads
    assert shape(512) == (1, True) and shape(1024) == (1, True)          # 128 and 256 blocks of two groups
    assert shape(2048) == (2, True)                                      # 512 blocks: all on the chip at once
    assert shape(2304) == (2, False) and shape(8192) == (2, False)       # one more round of blocks
    assert prefill_item_shape(100, 8, 64, 1, 256) == (1, True)           # a kernel with one group per item stays so
    # a kernel whose groups have waves of their own always gets two neighbouring groups
    split = lambda tokens: prefill_item_shape(tokens * 4, 8, 64, 2, 256, waves_split=True)
    assert split(64) == split(512) == split(2048) == split(8192) == (2, False)
    # every row still lands in exactly one item
    items = prefill_work_items([600], [37], 4, 0, 64, 1)
    rows = sorted(m0 for _, m0, other in items if other == -1)
    assert rows == list(range(0, 600 * 4, 64)) and all(other == -1 for _, _, other in items)
