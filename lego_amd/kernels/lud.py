"""Generator of the blocked LU decomposition kernels (no pivoting, in place).

Rodinia's LUD has three kernels per block step -- factor the diagonal block, solve the row and
column panels against it, update the trailing blocks -- and the reference uses LEGO for the last
one: a flat block of ``T*T`` threads is unfolded into a logical ``[R][T][R][T]`` thread structure
with ``OrderBy(Row(R*T, R*T)).GroupBy([(R, R), (T, T)], constraints).inv((ii*R + jj)*T*T + tid)``
so that each thread keeps an ``R x R`` register tile of results whose elements are ``T`` apart
(benchmarks/cuda/lud.py:5-12; kernels benchmarks/cuda/lud/lud_kernel_temp.cu:14-240, the LEGO
variant :297-352, host loop :358-390).

Here a block is 64 x 64, ``T = 16`` and ``R = 4`` (256 lanes per trailing block); the same
inverse places the lanes that stage the two panels in LDS, and the offsets of a block's elements
in the ``n x n`` matrix are those of ``OrderBy(Row(n, n)).TileBy([n/64, n/64], [64, 64])``.  The
product itself runs on the fp32 matrix cores, whose accumulator layout is one more LEGO
expression (``Row(4, 2, 4)``).  The diagonal block is eliminated by one wavefront with row ``t`` in
lane ``t``'s registers; a panel block is solved by one wavefront, a lane per column (row panel) or
per row (column panel), with the diagonal block's elements read across lanes.
"""
from __future__ import annotations

from ..lego import OrderBy, Row, le_constraint
from .common import BANNER, Emitted, code, idx, size, template, tidy

B, T, R = 64, 16, 4


def coarsening(ii, jj, tid):
    """``(i, j, ty, tx)`` of virtual thread ``(ii*R + jj)*T*T + tid``: register-tile coordinates
    and position inside the ``T x T`` lane grid (the reference's ``inv``, lud.py:8-12)."""
    constraints = [le_constraint(ii, R), le_constraint(jj, R), le_constraint(tid, T * T), le_constraint(0, tid)]
    lay = OrderBy(Row(R * T, R * T)).GroupBy([(R, R), (T, T)], constraints)
    return lay.inv((ii * R + jj) * T * T + tid)


def emit():
    n = size("n")
    bi, bj, r, c = (idx(s) for s in ("bi", "bj", "r", "c"))
    ii, jj, tid = (idx(s) for s in ("ii", "jj", "tid"))
    M = OrderBy(Row(n, n)).TileBy([n / B, n / B], [B, B])
    elem = tidy(M[bi, bj, r, c], {r: (0, B), c: (0, B), bi: (0, n / B), bj: (0, n / B)})
    i_e, j_e, ty_e, tx_e = (tidy(e, {ii: (0, R), jj: (0, R), tid: (0, T * T)}) for e in coarsening(ii, jj, tid))
    # the matrix core's accumulator: register q of lane l holds row Row(4, 2, 4)[q/4, l/32, q%4] of its 32 x 32 result
    q, l = idx("q"), idx("l")
    acc_row = tidy(OrderBy(Row(4, 2, 4)).TileBy([4, 2, 4])[q // 4, l // 32, q % 4], {q: (0, 16), l: (0, 64)})
    params = dict(
        banner=BANNER, B=B, T=T, R=R,
        matrix_layout=f"OrderBy(Row(n, n)).TileBy([n/{B}, n/{B}], [{B}, {B}])[bi, bj, r, c]",
        thread_layout=f"OrderBy(Row({R * T}, {R * T})).GroupBy([({R}, {R}), ({T}, {T})]).inv((ii*{R} + jj)*{T * T} + tid)",
        elem=code(elem), ci=code(i_e), cj=code(j_e), cty=code(ty_e), ctx=code(tx_e),
        acc_row=code(acc_row),
    )
    text = template("lud.hip.j2").render(**params)
    return Emitted("lud_f32.hip", text, ["lego_lud_f32_launch"]), dict(B=B)
