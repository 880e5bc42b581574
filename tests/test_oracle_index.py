"""Pins the CPU oracle's index maps: the offsets of the reference's generated transpose
programs, closed forms, and brute-force bijectivity; then checks that the product's
symbolic layouts evaluate to the oracle's numbers."""
import hashlib
import itertools
import json

import numpy as np
import pytest
import sympy as sp
from hypothesis import given, settings, strategies as st

import lego_amd as lg
from oracle import lego_index as li

TILE, BRX, BRY = 32, 8, 32


def oracle_transpose_accesses(kind, n):
    """Offsets of every access of the reference's transpose programs
    (benchmarks/mlir/transpose_naive.py:39-58, transpose_smem.py:46-80), shape
    ``[blocks, 256 threads, 4 steps]``, from the oracle's layouts."""
    nb = n // TILE
    bX = np.arange(nb * nb, dtype=np.int64)[:, None, None]
    tX = np.arange(256, dtype=np.int64)[None, :, None]
    it = np.arange(4, dtype=np.int64)[None, None, :]
    rby, rbx = li.tile_by(li.Order(li.row(nb, nb)), [nb, nb]).inv(bX)
    wby, wbx = li.tile_by(li.Order(li.col(nb, nb)), [nb, nb]).inv(bX)
    rty, rtx = li.tile_by(li.Order(li.row(BRX, BRY)), [BRX, BRY]).inv(tX)
    wty, wtx = li.tile_by(li.Order(li.col(BRY, BRX)), [BRY, BRX]).inv(tX)

    def tiled(inner):
        return li.tile_by(li.Order(li.row(n, n)), [nb, nb], [TILE // inner[0], TILE // inner[1]], inner)

    def staging(inner):
        return li.tile_by(li.Order(li.row(TILE, TILE)), [TILE // inner[0], TILE // inner[1]], inner)

    j, i = li.tile_by(li.Order(li.row(4, 1)), [4, 1]).inv(it)
    shape = (nb * nb, 256, 4)
    out = []
    if kind == "naive":
        out.append(tiled([BRX, BRY]).apply(rby, rbx, j, i, rty, rtx))
        out.append(tiled([BRY, BRX]).apply(wby, wbx, i, j, wty, wtx))
    else:
        out.append(tiled([BRX, BRY]).apply(rby, rbx, j, i, rty, rtx))
        out.append(staging([BRX, BRY]).apply(j, i, rty, rtx))
        j2, i2 = li.tile_by(li.Order(li.row(1, 4)), [1, 4]).inv(it)
        out.append(staging([BRY, BRX]).apply(j2, i2, wty, wtx))
        out.append(tiled([BRX, BRY]).apply(wby, wbx, i2, j2, rty, rtx))
    return [np.broadcast_to(a, shape).astype(np.int32) for a in out]


@pytest.mark.parametrize("kind", ["naive", "smem"])
def test_oracle_reproduces_reference_generated_offsets_256(kind, golden_dir):
    gold = np.load(golden_dir / "mlir_transpose_offsets.npz")
    keys = sorted(k for k in gold.files if k.startswith(f"{kind}_256_"))
    ours = oracle_transpose_accesses(kind, 256)
    assert len(keys) == len(ours)
    for key, arr in zip(keys, ours):
        assert np.array_equal(gold[key], arr), key


@pytest.mark.parametrize("kind,n", [(k, n) for k in ("naive", "smem") for n in (512, 1024, 2048)])
def test_oracle_reproduces_reference_generated_offset_digests(kind, n, golden_dir):
    digests = json.loads((golden_dir / "mlir_transpose_digests.json").read_text())
    ours = oracle_transpose_accesses(kind, n)
    keys = sorted(k for k in digests if k.startswith(f"{kind}_{n}_"))
    for key, arr in zip(keys, ours):
        assert hashlib.sha256(np.ascontiguousarray(arr).tobytes()).hexdigest() == digests[key]["sha256"], key


def test_golden_offsets_are_a_transpose(golden_dir):
    """The fixture itself moves element r*N+c to c*N+r (so it pins a transpose, not merely
    two arrays that agree with each other)."""
    gold = np.load(golden_dir / "mlir_transpose_offsets.npz")
    for kind in ("naive", "smem"):
        src = gold[f"{kind}_256_0_global_load"].astype(np.int64).ravel()
        dst = gold[[k for k in gold.files if k.startswith(f"{kind}_256_") and k.endswith("global_store")][0]]
        dst = dst.astype(np.int64).ravel()
        if kind == "smem":  # values pass through the staging tile: match store/load slots per block
            st_ = gold["smem_256_1_lds_store"].astype(np.int64)
            ld_ = gold["smem_256_2_lds_load"].astype(np.int64)
            src3 = gold["smem_256_0_global_load"].astype(np.int64)
            moved = np.empty_like(src3)
            for b in range(st_.shape[0]):
                tile = np.empty(1024, dtype=np.int64)
                tile[st_[b].ravel()] = src3[b].ravel()
                moved[b] = tile[ld_[b].ravel()].reshape(ld_[b].shape)
            src = moved.ravel()
        r, c = src // 256, src % 256
        assert np.array_equal(dst, c * 256 + r)
        assert len(np.unique(dst)) == 256 * 256


def test_closed_forms():
    src = li.tile_by(li.Order(li.row(4096, 4096)), [128, 128], [32, 32])
    dst = li.tile_by(li.Order(li.col(4096, 4096)), [128, 128], [32, 32])
    rng = np.random.default_rng(1)
    bi, bj = rng.integers(0, 128, 1000), rng.integers(0, 128, 1000)
    ti, tj = rng.integers(0, 32, 1000), rng.integers(0, 32, 1000)
    assert np.array_equal(src.apply(bi, bj, ti, tj), 131072 * bi + 32 * bj + 4096 * ti + tj)
    assert np.array_equal(dst.apply(bi, bj, ti, tj), 131072 * bj + 32 * bi + 4096 * tj + ti)
    # a permutation block is numpy's transpose of strides
    p = li.Perm((3, 4, 5), [2, 0, 1])
    ref = np.arange(60).reshape(5, 3, 4)    # stored order: axis 2, axis 0, axis 1
    for idx in itertools.product(range(3), range(4), range(5)):
        assert p.apply(idx) == ref[idx[2], idx[0], idx[1]]
        assert p.inv(p.apply(idx)) == idx
    # the five-dimensional permutation of benchmarks/examples/graphene.py:5-7
    g = li.Layout([2] * 5, [li.Order(li.Perm([2] * 5, [4, 1, 3, 2, 0]))])
    for i, j, k, w, q in itertools.product(range(2), repeat=5):
        assert g.apply(i, j, k, w, q) == i + 8 * j + 2 * k + 16 * q + 4 * w


small = st.integers(min_value=1, max_value=4)


@settings(max_examples=60, deadline=None)
@given(st.lists(small, min_size=1, max_size=3), st.lists(small, min_size=1, max_size=3), st.randoms())
def test_tiled_layouts_are_bijections_and_product_agrees(tiles, inner, rnd):
    rank = min(len(tiles), len(inner))
    tiles, inner = tiles[:rank], inner[:rank]
    full = [t * i for t, i in zip(tiles, inner)]
    perm = list(range(rank))
    rnd.shuffle(perm)
    oracle = li.tile_by(li.Order(li.Perm(full, perm)), tiles, inner)
    product = lg.OrderBy(lg.RegP(full, perm)).TileBy(tiles, inner)
    seen = set()
    for idx in itertools.product(*[range(n) for n in tiles + inner]):
        off = oracle.apply(*idx)
        assert 0 <= off < oracle.size()
        assert oracle.inv(off) == idx
        assert product.apply(*idx) == off                       # raw product map, integers
        assert tuple(product.inv_raw(off)) == idx
        seen.add(off)
    assert len(seen) == oracle.size()
    # the simplified symbolic offset evaluates to the same numbers
    names = sp.symbols(f"x0:{2 * rank}", integer=True, nonnegative=True)
    expr = product[tuple(names)]
    f = sp.lambdify(names, expr, modules=[{"floor": np.floor, "Mod": np.mod}, "numpy"])
    for idx in itertools.islice(itertools.product(*[range(n) for n in tiles + inner]), 64):
        assert int(f(*idx)) == oracle.apply(*idx)
    # and so does the simplified inverse
    flat = sp.Symbol("flat", integer=True, nonnegative=True)
    inv = product.inv(flat)
    for off in range(min(oracle.size(), 64)):
        got = tuple(int(c.subs(flat, off)) for c in inv)
        assert got == oracle.inv(off)


def test_two_block_order_by():
    o = li.tile_by(li.Order(li.row(3, 2), li.col(2, 4)), [3, 2], [2, 4])
    p = lg.OrderBy(lg.Row(3, 2), lg.Col(2, 4)).TileBy([3, 2], [2, 4])
    seen = set()
    for idx in itertools.product(range(3), range(2), range(2), range(4)):
        # tiles row-major, inside a tile column-major
        want = (idx[0] * 2 + idx[1]) * 8 + idx[3] * 2 + idx[2]
        assert o.apply(*idx) == want == p.apply(*idx)
        seen.add(want)
    assert len(seen) == 48
