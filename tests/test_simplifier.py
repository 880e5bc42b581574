"""simplify_ops preserves values: for random in-range integer assignments the simplified
expression evaluates to what the raw one does (that is its whole contract), and it removes
the floor/Mod nests that tiling produces."""
import random

import pytest
import sympy as sp
from sympy import Mod, floor

import lego_amd as lg
from lego_amd.simplifier import BitXor, RangeProver, simplify_ops


def _evaluate(expr, env):
    val = expr.xreplace({k: sp.Integer(v) for k, v in env.items()})
    assert val.is_Integer, val
    return int(val)


CASES = [
    # (layout factory, key builder, sizes)
    ("tile2", lambda M, K, BM, BK: lg.OrderBy(lg.Row(M, K)).TileBy([M / BM, K / BK], [BM, BK]), 4),
    ("tile2col", lambda M, K, BM, BK: lg.OrderBy(lg.Col(M, K)).TileBy([M / BM, K / BK], [BM, BK]), 4),
]


@pytest.mark.parametrize("name,factory,rank", CASES)
def test_symbolic_tile_offsets_preserve_values(name, factory, rank):
    M, K, BM, BK = sp.symbols("M K BM BK", integer=True, positive=True)
    lay = factory(M, K, BM, BK)
    a, b, c, d = sp.symbols("a b c d", integer=True, nonnegative=True)
    simplified = lay[a, b, c, d]
    raw = lay.apply(a, b, c, d)
    assert not simplified.has(floor) and not simplified.has(Mod)
    rng = random.Random(0)
    for _ in range(50):
        bm, bk = rng.choice([1, 2, 4, 8]), rng.choice([1, 2, 4, 16])
        m, k = bm * rng.randint(1, 5), bk * rng.randint(1, 5)
        env = {M: m, K: k, BM: bm, BK: bk, a: rng.randrange(m // bm), b: rng.randrange(k // bk),
               c: rng.randrange(bm), d: rng.randrange(bk)}
        assert _evaluate(simplified, env) == _evaluate(sp.sympify(raw), env)


def test_random_floor_mod_expressions_preserve_values():
    rng = random.Random(1)
    x, y, z = sp.symbols("x y z", integer=True, nonnegative=True)
    for trial in range(60):
        nx, ny, nz = (rng.choice([2, 3, 4, 8, 16]) for _ in range(3))
        c1, c2, d1, d2 = (rng.choice([1, 2, 3, 4, 8, 12, 16, 32]) for _ in range(4))
        inner = c1 * x + c2 * y + z
        expr = rng.choice([
            floor(inner / d1) * d2 + Mod(inner, d1),
            Mod(floor(inner / d1), d2) + d1 * floor(inner / (d1 * d2)),
            floor((d1 * x + Mod(y, d1)) / d1) + Mod(d2 * z + Mod(x, d2), d2),
            Mod(Mod(inner, d1 * d2), d1) + floor(Mod(inner, d1) / d1),
            BitXor(Mod(inner, 16), 4 * Mod(floor(x / 1), 4)) + floor(inner / 16) * 16,
        ])
        out = simplify_ops(expr, {x: (0, nx), y: (0, ny), z: (0, nz)})
        for _ in range(20):
            env = {x: rng.randrange(nx), y: rng.randrange(ny), z: rng.randrange(nz)}
            assert _evaluate(out, env) == _evaluate(expr, env), (expr, out, env)


def test_prover_is_sound_on_obvious_cases():
    i, j = sp.symbols("i j", integer=True)
    n, m = sp.symbols("n m", integer=True, positive=True)
    p = RangeProver({i: (0, n), j: (0, m)})
    assert p.less(i * m + j, n * m)             # a mixed-radix number is below its radix product
    assert p.nonneg(i * m + j)
    assert not p.less(i * m + j + 1, n * m)     # off by one must not be "proven"
    assert not p.less(i * (m + 1), n * m)
    assert p.can_prove(sp.StrictLessThan(floor((i * m + j) / m), n, evaluate=False))
    assert not p.can_prove(sp.StrictLessThan(i, n - 1, evaluate=False))


def test_grouped_order_needs_its_lemma_and_stays_sound():
    npm, npn, gm, pid = sp.symbols("npm npn gm pid", integer=True, positive=True)
    lay = lg.OrderBy(lg.Col(sp.Max(npm // gm, 1), 1), lg.Col(sp.Min(npm, gm), npn)).TileBy([npm, npn])
    pm, pn = lay.inv(pid)
    raw_m, raw_n = lay.inv_raw(pid)
    for a, b, c in [(8, 4, 2), (8, 4, 4), (4, 3, 8), (6, 5, 3), (12, 2, 4), (1, 1, 8)]:
        for v in range(a * b):
            env = {npm: a, npn: b, gm: c, pid: v}
            assert _evaluate(pm, env) == _evaluate(sp.sympify(raw_m), env)
            assert _evaluate(pn, env) == _evaluate(sp.sympify(raw_n), env)
