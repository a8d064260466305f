"""The host-side launch rules of the grouped-product kernels, checked without a GPU through the
library's launch planner (mi_moe_debug_plan_*: says what would be launched, launches nothing).

A launch is refused by the library itself when the LDS size its rules worked with differs from what the
chosen variant's own layout needs for the values it is given, or does not fit a CU: a sweep that meets
no refusal shows that the two sides agree on every shape swept."""
import itertools
import random

import pytest

from variant_cases import BLOCK_CASES, OP_CASE


@pytest.fixture(scope="module")
def capi():
    import mlx_rs_amd as m
    m.load_library()
    return m.capi


def test_every_variant_is_listed(capi):
    names = capi.kernel_launches()
    assert len(names) == 67, sorted(names)
    assert sum(n.startswith("qmm_large_kernel") for n in names) == 12


def test_the_case_table_reaches_every_variant(capi):
    want = set(capi.kernel_launches())
    got = {OP_CASE["variant"]}
    for (H, I, E, k, T, bits), names in BLOCK_CASES:
        plan = [n for n, _ in capi.plan_forward(capi.Config(H, E, k, I, bits, 64, 0), T)]
        for n in names:
            assert n in plan, ((H, I, E, k, T, bits), n, plan)
        got.update(names)
    c = OP_CASE
    plan = [n for n, _ in capi.plan_grouped(c["N"], c["K"], c["bits"], False, c["rows"], 1, c["rows"])]
    assert plan == [c["variant"]]
    assert got == want, sorted(want - got)


def test_no_shape_of_a_sweep_is_refused(capi):
    """Grid and LDS of every planned launch fit the chip; nothing is refused (20 000 random extents)."""
    rng = random.Random(4)
    n = 0
    for _ in range(20000):
        bits = rng.choice((4, 8))
        glu = rng.choice((False, True))
        N = 16 * rng.choice((1, 2, 3, 4, 6, 8, 12, 16, 24, 32, 48, 64, 96, 128, 192, 256, 896))
        K = rng.choice((512 * rng.randint(1, 27), (128 if bits == 4 else 64) * rng.randint(1, 100)))
        act = rng.choice((1, 1, 2, 3, 4, 5, 6, 8, 12, 16, 24, 32, 64, 128, 256, 512))
        rpe = rng.choice((1, 1, 2, 3, 4, 5, 6, 7, 8, 9, 10, 12, 16, 17, 20, 24, 32, 48, 64))
        total = act * rpe
        longest = min(total, rpe * rng.choice((1, 2, 4, 16, 512)))
        tiled = rng.choice((False, True))
        for name, info in capi.plan_grouped(N, K, bits, glu, total, act, longest, rng.choice((8, 16)) if tiled else 0,
                                            tiled, bits == 4 and glu):
            gx, gy = (int(v) for v in info["grid"].split("x"))
            assert 1 <= gx and 1 <= gy <= 65535 and int(info["lds"]) <= 160 * 1024, (name, info)
            n += 1
    assert n >= 20000


def test_rows_too_long_for_a_cu_are_refused_with_a_message(capi):
    # gate and up rows of 16256 4-bit values in whole rows (no slabs: not a multiple of 512) with their scale
    # tiles need more LDS than a CU has
    with pytest.raises(capi.MoeError):
        capi.plan_grouped(384, 16256, 4, True, 48, 12, 16)
