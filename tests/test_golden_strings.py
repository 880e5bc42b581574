"""The product's layout algebra + printers reproduce, character for character, the offset
expressions the reference committed in its generated kernels; and those same strings,
evaluated numerically, agree with the CPU oracle's index maps (which pins the oracle)."""
import json
import types

import numpy as np
import pytest
import sympy as sp

from lego_amd.lego_c import LEGOCCodePrinter
from lego_amd.lego_python import (Col, GenP, LEGOPythonCodePrinter, OrderBy, Row, antidiag,
                                  divisibility_constraint, get_arange, le_constraint)
from oracle import lego_index as li

P = dict(integer=True, positive=True)


def _matmul_syms():
    return sp.symbols("M N K BM BN BK num_pid_m num_pid_n GM pid k", **P)


def build(layout):
    """The LEGO source of each golden entry (reference file:line in the docstrings)."""
    M, N, K, BM, BN, BK, npm, npn, GM, pid, k = _matmul_syms()
    if layout.startswith("matmul_A"):      # benchmarks/triton/matmul_sympy.py:37-40
        order = Col(M, K) if layout.endswith("col") else Row(M, K)
        return OrderBy(order).TileBy([M / BM, K / BK], [BM, BK])["pid_m", k, :, :]
    if layout.startswith("matmul_B"):      # matmul_sympy.py:43-46
        order = Col(K, N) if layout.endswith("col") else Row(K, N)
        return OrderBy(order).TileBy([K / BK, N / BN], [BK, BN])[k, "pid_n", :, :]
    if layout == "matmul_C":               # matmul_sympy.py:49-54
        return OrderBy(Row(M, N)).TileBy([M / BM, N / BN], [BM, BN])["pid_m", "pid_n", :, :]
    if layout in ("matmul_pid_m", "matmul_pid_n"):  # matmul_sympy.py:57-65
        L = OrderBy(Col(sp.Max(npm // GM, 1), 1), Col(sp.Min(npm, GM), npn)).TileBy([npm, npn])
        return L.inv(pid)[0 if layout.endswith("m") else 1]
    if layout == "softmax_row":            # benchmarks/triton/softmax_sympy.py:6-8
        n_rows, n_cols, BS = sp.symbols("n_rows n_cols BLOCK_SIZE", **P)
        return OrderBy(Row(n_rows, n_cols)).TileBy([n_rows, n_cols])["row_idx", get_arange(0, BS)]
    if layout.startswith("layernorm"):     # benchmarks/triton/layernorm_triton.py:7-23
        M_, N_, BSN = sp.symbols("M N BLOCK_SIZE_N", **P)
        X_L = OrderBy(Row(M_, N_)).TileBy([M_, N_ / BSN], [1, BSN],
                                          user_constraints=[divisibility_constraint(N_, BSN)])
        return {
            "layernorm_xy": lambda: X_L["pid", "k", 0, :],
            "layernorm_cols": lambda: X_L[0, "k", 0, :],
            "layernorm_w": lambda: OrderBy(Row(M_)).TileBy([M_])["pid",],
            "layernorm_xy_bwd": lambda: X_L["pid", 0, 0, :],
            "layernorm_dwdb_bwd": lambda: X_L["lock_id", 0, 0, :],
            "layernorm_w_bwd": lambda: OrderBy(Row(BSN)).TileBy([BSN])[:,],
        }[layout]()
    if layout.startswith("grouped"):       # benchmarks/triton/grouped_gemm_sympy.py:7-24,38-39
        gm, gn, gk, BM_, BN_, BK_ = sp.symbols("gm gn gk BLOCK_SIZE_M BLOCK_SIZE_N BLOCK_SIZE_K", **P)
        if layout == "grouped_A":
            return OrderBy(Row(gm, gk)).TileBy([gm / BM_, gk / BK_], [BM_, BK_])["tile_m_idx", "kk", :, :]
        if layout == "grouped_B":
            return OrderBy(Row(gk, gn)).TileBy([gk / BK_, gn / BN_], [BK_, BN_])["kk", "tile_n_idx", :, :]
        return OrderBy(Row(gm, gn)).TileBy([gm / BM_, gn / BN_], [BM_, BN_])["tile_m_idx", "tile_n_idx", :, :]
    if layout.startswith("bricks"):        # benchmarks/cuda/bricks_f3d.py:7-21
        i, j, k_, idf, jdf, kdf, bx, by, bz = sp.symbols("i j k i_diff j_diff k_diff bx by bz", **P)
        n, b = 384, 8
        lay = (OrderBy(Row(n, n, n)) if "normal" in layout
               else OrderBy(Row(n // b, n // b, n // b), Row(b, b, b))).TileBy([n // b] * 3, [b] * 3)
        if layout.endswith("halo"):
            return lay[bx, by, bz, i + idf, j + jdf, k_ + kdf]
        return lay[bx, by, bz, i, j, k_]
    if layout.startswith("lud"):           # benchmarks/cuda/lud.py:5-12
        R, T, ii, jj, tid = sp.symbols("R T ii jj tid", **P)
        cons = [le_constraint(ii, R), le_constraint(jj, R), le_constraint(tid, T * T), le_constraint(0, tid)]
        res = OrderBy(Row(R * T, R * T)).GroupBy([(R, R), (T, T)], cons).inv((ii * R + jj) * T * T + tid)
        return res[["lud_i", "lud_j", "lud_ty", "lud_tx"].index(layout)]
    if layout == "nw_antidiag":            # benchmarks/cuda/nw_sympy.py:6-11
        n, i, j = sp.symbols("n i j", integer=True)
        return OrderBy(GenP([n, n], lambda x: antidiag(n, x), None)).TileBy((n, n))[i, j]
    raise KeyError(layout)


def entries(golden_dir=None):
    from conftest import GOLDEN
    return json.loads((GOLDEN / "reference_strings.json").read_text())["entries"]


def printer_for(kind):
    if kind == "python":
        return LEGOPythonCodePrinter(allow_unknown_functions=True)
    if kind == "python_nobroadcast":
        return LEGOPythonCodePrinter(allow_unknown_functions=True, do_broadcast=False)
    return LEGOCCodePrinter()


@pytest.mark.parametrize("entry", entries(), ids=lambda e: e["layout"])
def test_product_prints_reference_text(entry):
    # the generators print sp.simplify(expr) (benchmarks/triton/matmul_sympy.py:454)
    text = printer_for(entry["printer"]).doprint(sp.simplify(build(entry["layout"])))
    assert text == entry["text"], entry["source"]


# ---- the same strings, as numbers, against the oracle --------------------------------

def _eval(text, **names):
    tl = types.SimpleNamespace(arange=lambda lo, hi: np.arange(lo, hi, dtype=np.int64))
    return eval(text, {"tl": tl, "min": min, "max": max, "__builtins__": {}}, names)


def _text(layout):
    return next(e["text"] for e in entries() if e["layout"] == layout)


@pytest.mark.parametrize("order", ["row", "col"])
def test_oracle_matches_matmul_operand_strings(order):
    M, N, K, BM, BN, BK = 96, 64, 80, 32, 16, 8
    a = li.tile_by(li.Order((li.row if order == "row" else li.col)(M, K)), [M // BM, K // BK], [BM, BK])
    b = li.tile_by(li.Order((li.row if order == "row" else li.col)(K, N)), [K // BK, N // BN], [BK, BN])
    c = li.tile_by(li.Order(li.row(M, N)), [M // BM, N // BN], [BM, BN])
    for pid_m in range(M // BM):
        for k in range(K // BK):
            want = _eval(_text(f"matmul_A_{order}"), M=M, K=K, BM=BM, BK=BK, pid_m=pid_m, k=k)
            got = a.apply(pid_m, k, np.arange(BM)[:, None], np.arange(BK)[None, :])
            assert np.array_equal(want, got)
    for pid_n in range(N // BN):
        for k in range(K // BK):
            want = _eval(_text(f"matmul_B_{order}"), N=N, K=K, BN=BN, BK=BK, pid_n=pid_n, k=k)
            got = b.apply(k, pid_n, np.arange(BK)[:, None], np.arange(BN)[None, :])
            assert np.array_equal(want, got)
    want = _eval(_text("matmul_C"), M=M, N=N, BM=BM, BN=BN, pid_m=2, pid_n=3)
    assert np.array_equal(want, c.apply(2, 3, np.arange(BM)[:, None], np.arange(BN)[None, :]))


@pytest.mark.parametrize("npm,npn,gm", [(32, 32, 8), (32, 32, 4), (16, 8, 8), (8, 16, 8), (4, 4, 8), (6, 5, 3)])
def test_oracle_matches_grouped_pid_strings(npm, npn, gm):
    G, g = max(npm // gm, 1), min(npm, gm)
    lay = li.tile_by(li.Order(li.col(G, 1), li.col(g, npn)), [npm, npn])
    pid = np.arange(npm * npn, dtype=np.int64)
    want_m = _eval(_text("matmul_pid_m"), pid=pid, GM=gm, num_pid_m=npm, num_pid_n=npn)
    want_n = _eval(_text("matmul_pid_n"), pid=pid, GM=gm, num_pid_m=npm, num_pid_n=npn)
    got_m, got_n = lay.inv(pid)
    assert np.array_equal(want_m, got_m) and np.array_equal(want_n, got_n)
    # and both equal the textbook grouped order of the Triton tutorial kernel
    from oracle.kernels import grouped_pid
    tm, tn = grouped_pid(pid, npm, npn, gm)
    assert np.array_equal(tm, got_m) and np.array_equal(tn, got_n)
    # a bijection onto the tile grid
    assert len(set(zip(got_m.tolist(), got_n.tolist()))) == npm * npn


def test_oracle_matches_bricks_strings():
    rng = np.random.default_rng(0)
    bx, by, bz = (rng.integers(0, 48, 200) for _ in range(3))
    i, j, k = (rng.integers(0, 8, 200) for _ in range(3))
    normal = li.tile_by(li.Order(li.row(384, 384, 384)), [48] * 3, [8] * 3)
    bricks = li.tile_by(li.Order(li.row(48, 48, 48), li.row(8, 8, 8)), [48] * 3, [8] * 3)
    names = dict(bx=bx, by=by, bz=bz, i=i, j=j, k=k)
    assert np.array_equal(_eval(_text("bricks_normal"), **names), normal.apply(bx, by, bz, i, j, k))
    assert np.array_equal(_eval(_text("bricks_bricks"), **names), bricks.apply(bx, by, bz, i, j, k))


def test_oracle_matches_row_strings():
    n_rows, n_cols = 7, 24
    lay = li.tile_by(li.Order(li.row(n_rows, n_cols)), [n_rows, n_cols])
    for r in range(n_rows):
        want = _eval(_text("softmax_row"), n_cols=n_cols, row_idx=r, BLOCK_SIZE=n_cols)
        assert np.array_equal(want, lay.apply(r, np.arange(n_cols)))
    M, N, BN = 5, 48, 16
    x = li.tile_by(li.Order(li.row(M, N)), [M, N // BN], [1, BN])
    for pid in range(M):
        for k in range(N // BN):
            want = _eval(_text("layernorm_xy"), N=N, BLOCK_SIZE_N=BN, pid=pid, k=k)
            assert np.array_equal(want, x.apply(pid, k, 0, np.arange(BN)))


def test_oracle_matches_lud_strings():
    R, T = 3, 4
    lay = li.Layout([R, R, T, T], [li.Order(li.row(R * T, R * T))])
    for ii in range(R):
        for jj in range(R):
            for tid in range(T * T):
                got = lay.inv((ii * R + jj) * T * T + tid)
                assert got == (ii, jj, tid // T, tid % T)
