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

from ..lego import Col, OrderBy, Row, le_constraint
from .common import BANNER, Emitted, code, idx, size, template, tidy

B, T, R = 64, 16, 4
# side (in blocks) of the trailing square from which the next panels are solved on a second stream meanwhile
AHEAD_MIN = 72
# the trailing square is walked in groups of GROUP block rows, column by column inside a group (the grouped launch
# order of the reference's matmul, matmul_sympy.py:57-65), and each of the XCDS L2 caches gets a contiguous run of it
GROUP, XCDS = 8, 8
# a workgroup takes a run of up to GROUP blocks of a column as long as that leaves this many workgroups (two per CU, twice)
MIN_WGS = 1024


def block_order(ng, q, nsub, pid):
    """``(group, column, part)`` of position ``pid`` in the walk over ``ng`` groups of ``GROUP`` block rows: column
    by column inside a group, a column of a group in ``nsub`` parts, one workgroup per part (parts past the
    square, in the last group, are skipped by the kernel)."""
    return OrderBy(Row(ng, q, nsub)).TileBy([ng, q, nsub]).inv(pid)


def xcd_remap(per, wg):
    """Workgroup id -> position such that the ids one XCD receives (``wg % XCDS``) form a contiguous run of
    ``per`` positions: ``wg`` read as ``(j, x)`` of a row-major ``[per, XCDS]`` box, stored column-major."""
    j, x = OrderBy(Row(per, XCDS)).TileBy([per, XCDS]).inv(wg)
    return OrderBy(Col(per, XCDS)).TileBy([per, XCDS])[j, x]


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
    ng, qq, per, pid, wg = size("ng"), size("q"), size("per"), idx("pid"), idx("wg")
    nsub = size("nsub")
    og, oc, osub = (tidy(e, {pid: (0, ng * qq * nsub)}) for e in block_order(ng, qq, nsub, pid))
    xcd_pid = tidy(xcd_remap(per, wg), {wg: (0, per * XCDS)})
    # k of the j-th matrix-core instruction in lane l: Row(2, 32)[l/32, j] (halves of the wavefront take halves of k)
    j = idx("j")
    k_of_lane = tidy(OrderBy(Row(2, B // 2)).TileBy([2, B // 2])[l // 32, j], {l: (0, 64), j: (0, B // 2)})
    params = dict(
        banner=BANNER, B=B, T=T, R=R, AHEAD_MIN=AHEAD_MIN,
        matrix_layout=f"OrderBy(Row(n, n)).TileBy([n/{B}, n/{B}], [{B}, {B}])[bi, bj, r, c]",
        thread_layout=f"OrderBy(Row({R * T}, {R * T})).GroupBy([({R}, {R}), ({T}, {T})]).inv((ii*{R} + jj)*{T * T} + tid)",
        elem=code(elem), ci=code(i_e), cj=code(j_e), cty=code(ty_e), ctx=code(tx_e),
        acc_row=code(acc_row), k_of_lane=code(k_of_lane), k_layout=f"Row(2, {B // 2})[l/32, j]", GROUP=GROUP, XCDS=XCDS,
        order_g=code(og), order_c=code(oc), order_sub=code(osub), xcd_pid=code(xcd_pid), MIN_WGS=MIN_WGS,
        order_layout="OrderBy(Row(ng, q, nsub)).TileBy([ng, q, nsub]).inv(pid) -> (group, column, part)",
        xcd_layout=f"OrderBy(Col(per, {XCDS})).TileBy([per, {XCDS}])[Row(per, {XCDS}).inv(wg)]",
    )
    text = template("lud.hip.j2").render(**params)
    return Emitted("lud_f32.hip", text, ["lego_lud_f32_launch", "lego_lud_f32_plan"]), dict(B=B)
