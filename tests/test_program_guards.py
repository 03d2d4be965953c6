"""The conditions of a step program's operations (engine/program.Guard): and, or, not against brute force."""
import itertools
import random

from infernum_amd.engine.program import ALWAYS, NEVER, Guard, Var


def _random_guard(rng, vars_):
    g = NEVER
    for _ in range(rng.randint(1, 3)):
        c = ALWAYS
        for _ in range(rng.randint(1, 3)):
            v = rng.choice(vars_)
            if rng.random() < 0.5:
                lo = rng.randint(-5, 150)
                c = c & Guard.between(v, lo if rng.random() < 0.8 else None, lo + rng.randint(0, 60) if rng.random() < 0.8 else None)
            else:
                c = c & Guard.blocks(v, rng.randrange(512))
        g = g | c
    return g


def test_and_or_not_against_brute_force():
    rng = random.Random(3)
    a, b = Var(0, "a"), Var(1, "b")
    points = [(x, y) for x in (-3, 0, 1, 15, 16, 17, 33, 64, 65, 100, 128, 129, 145, 300) for y in (0, 1, 16, 17, 129, 200)]
    for _ in range(300):
        g, h = _random_guard(rng, [a, b]), _random_guard(rng, [a, b])
        for p in points:
            assert (g & h).holds(p) == (g.holds(p) and h.holds(p))
            assert (g | h).holds(p) == (g.holds(p) or h.holds(p))
            assert (~g).holds(p) == (not g.holds(p))


def test_always_never_and_blocks():
    n = Var(0, "n")
    assert ALWAYS.holds([5]) and not NEVER.holds([5]) and (~ALWAYS).never and not (~NEVER).never
    first_two = Guard.blocks(n, 0b11)
    assert [x for x in range(-1, 40) if first_two.holds([x])] == list(range(1, 33))
    above = Guard.blocks(n, 1 << 8)
    assert not above.holds([128]) and above.holds([129]) and above.holds([10 ** 6])
    # a range that rules every block out leaves nothing
    assert (Guard.blocks(n, 0b1) & Guard.between(n, 17, 40)).never
    assert (Guard.between(n, 3, 2)).never
    # a multiple of a number is an argument, not something a condition can be about
    import pytest
    from infernum_amd.engine.program import ProgramError
    with pytest.raises(ProgramError):
        Guard.between(2 * n, 0, 1)
    assert (3 * n + 2).mul == 3 and (3 * n + 2).add == 2 and ((n + 2) * 3).add == 6


def test_the_product_plan_covers_every_number_of_rows_once(monkeypatch):
    """parts/linear.plan: whatever the weight and use, every block of rows has exactly one route."""
    import importlib
    import torch
    L = importlib.import_module("infernum_amd.parts.linear")
    # the number of parts of a split product is the kernel library's to say; any rule serves here
    monkeypatch.setattr(L.K, "gemm_skinny_splits", lambda N, K: 4 if N < 8192 else 1)
    monkeypatch.setitem(L.KNOWN_MID_ROWS, (48, 4096), ((129, 256, 3), (257, 300, 2)))      # beside the shapes the table holds
    try:
        for N, Kd in itertools.product((48, 4096, 28672, 16385), (64, 4096, 100, 14336)):
            for dtype, out, epi, keep, kernels in itertools.product(
                    (torch.float32, torch.bfloat16), (torch.float32, torch.bfloat16), (None, "swiglu"), (False, True),
                    ("auto", "generic")):
                if dtype == torch.bfloat16 and out == torch.float32 and epi and kernels == "auto" and Kd % 8 == 0:
                    continue                                   # refused with a clear error, see below
                for route in ("table", "static"):
                    L.set_gemm_route(route)
                    seen = 0
                    for r in L.plan(N, Kd, dtype, out, epi, keep, kernels):
                        if r.rows is not None:                 # a route for a range of rows: ahead of the one it takes from
                            assert r.blocks == L.ALL_BLOCKS and 1 <= r.rows[0] <= r.rows[1] and not seen
                            assert (r.kind == "mfma_split" and r.parts >= 1 and keep and epi is None) or \
                                (r.kind == "mfma_f32" and out == torch.float32 and dtype == torch.bfloat16) or \
                                (r.kind == "mfma_swiglu" and epi == "swiglu")
                            continue
                        assert r.blocks and not (seen & r.blocks)
                        seen |= r.blocks
                    assert seen == L.ALL_BLOCKS
                    for M in (1, 16, 17, 64, 65, 128, 129, 200, 256, 257, 5000):
                        assert L.route_of(L.plan(N, Kd, dtype, out, epi, keep, kernels), M) is not None
    finally:
        L.set_gemm_route("table")
