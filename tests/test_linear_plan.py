"""The plans ``linear`` makes for bfloat16 products at few rows, checked on the host against what
the kernels accept (the checks of ``gemm_skinny``, ``gemm_tile64`` and their entry points), over a
grid of sizes that includes those of real models and sizes that share out unevenly."""
import itertools

import pytest

from jax_vllm_amd.ops import kernels as K

ROWS = [1, 2, 3, 8, 9, 16, 17, 32, 33, 64, 65, 200]
WIDTHS = [16, 64, 520, 1024, 2048, 2560, 4096, 5120, 6144, 7168, 8192, 8200, 10240, 24576, 34816, 51200, 151936]
INNER = [8, 256, 264, 512, 1000, 1024, 1536, 2048, 2560, 3072, 4096, 5120, 6152, 8192, 9728, 12288, 17408, 25600]


def acceptable(m, n, k, silu, plan):
    """What the kernel entry points would say to this plan."""
    shape, parts = plan
    if parts > 1 and silu:
        return "no activation of partial sums"
    if shape == K.TILE64:
        rounds = -(-k // 256)
        if m > 64 or (parts > 1 and -(-rounds // parts) * (parts - 1) >= rounds):
            return "a group of 64-row blocks without columns"
        return None
    if m > 64:
        return "more than 64 rows"
    kind, a, b = shape
    if kind == -2:
        if (16 < m <= 32 and b not in K.STAY_PIECES_32_ROWS) or (m > 32 and b > 5) or b not in K.STAY_PIECES or a < 1 or \
                not (256 * b * (parts - 1) < k <= 256 * b * parts):
            return "staying blocks that do not cover the inner size"
    elif kind == -1:
        phases = -(-k // (a * b * 32))
        if m > 16 or silu or (parts > 1 and -(-phases // parts) * (parts - 1) >= phases):
            return "a group of resident-x blocks without columns"
    elif shape != (0, 0, 0):
        return "unknown block shape"
    return None


@pytest.mark.parametrize("silu,partial_ok", [(False, False), (False, True), (True, False)])
def test_every_plan_is_one_the_kernels_accept(silu, partial_ok):
    for m, n, k in itertools.product(ROWS, WIDTHS, INNER):
        plan = K.streaming_plan(m, n, k, gate_pairs=silu, partial_ok=partial_ok)
        if plan is None:
            continue                        # the library's
        assert m <= 64 and k % 8 == 0
        assert plan[1] == 1 or partial_ok, (m, n, k, plan)
        why = acceptable(m, n, k, silu, plan)
        assert why is None, f"{(m, n, k)}: {plan}: {why}"
        if plan[1] > 1:                     # the readers of partial products take 2..4 parts of limited width
            assert 2 <= plan[1] <= 4 and n % 4 == 0 and n <= K.PARTIAL_SUM_MAX_WIDTH


def test_plans_at_the_sizes_they_were_measured_at():
    plan = K.streaming_plan
    assert plan(8, 4096, 4096, partial_ok=True) == ((-2, 512, 4), 4)            # o_proj, 8B
    assert plan(8, 4096, 12288, partial_ok=True) == ((-2, 256, 12), 4)          # down_proj, 8B
    assert plan(8, 24576, 4096, gate_pairs=True) == ((-2, 256, 16), 1)          # gate and up, 8B
    assert plan(64, 4096, 12288, partial_ok=True) == (K.TILE64, 4)              # down_proj at 64 rows
    assert plan(24, 24576, 4096, gate_pairs=True) == ((-2, 256, 16), 1)         # gate and up at 17..32 rows: W in slots
    assert plan(32, 151936, 4096) == ((-2, 256, 16), 1)                         # the output embedding likewise
    assert plan(33, 24576, 4096, gate_pairs=True) is None                       # beyond: the library
    assert plan(24, 34816, 5120, gate_pairs=True) is None                       # 20 pieces a wave do not fit beside two row tiles
    assert plan(64, 5120, 17408, partial_ok=True) == (K.TILE64, 3)              # 80 tiles of 64 rows: 3 groups fill 256 units
    assert plan(64, 4096, 4096, partial_ok=True) == ((-2, 256, 4), 4)           # four row tiles of x in registers
    assert plan(64, 5120, 8192, partial_ok=True) is None                        # 8 pieces a wave: too many registers for that
    assert plan(32, 4096, 4096, partial_ok=True) == ((-2, 256, 4), 4)           # two row tiles of x in registers
    assert plan(12, 5120, 17408, partial_ok=True) == ((-2, 256, 17), 4)         # where the library collapses
    assert plan(8, 1024, 3072, partial_ok=True) == ((-2, 512, 8), 2)            # no piece count covers 3,072 with 4 groups
    assert plan(8, 5120, 25600, partial_ok=True) == (K.PARTIAL_SHAPE, 4)        # none with 2 or 4: x resident in LDS
    assert plan(8, 1024, 1000 * 8, partial_ok=True)[1] in (2, 3, 4)
    assert plan(8, 34816, 5120, gate_pairs=True) == ((-2, 256, 20), 1)          # gate and up, 14B
    assert plan(1, 24576, 4096, gate_pairs=True) == ((-2, 256, 16), 1)          # one row: the same blocks
    assert plan(8, 10240, 5120, partial_ok=True) == ((0, 0, 0), 1)              # wider than the norm adds parts of ...
    assert plan(8, 10240, 5120, partial_ok=True, partial_max_width=None) == ((-2, 256, 5), 4)   # ... but the rotation kernel does
    assert plan(8, 4096, 4100) is None                                          # inner size no multiple of 8
