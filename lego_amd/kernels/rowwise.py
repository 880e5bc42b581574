"""Generator of the row softmax and LayerNorm-forward kernels.

The reference's kernels take one LEGO offset vector per row,
``n_cols*row_idx + tl.arange(0, BLOCK_SIZE)`` (benchmarks/triton/softmax_sympy.py:6-19) and
``BLOCK_SIZE_N*k + N*pid + tl.arange(0, BLOCK_SIZE_N)``
(benchmarks/triton/layernorm_triton.py:10-19), and let Triton decide what a lane loads.
Here the lane's share is part of the layout: a row is a ``[vectors, 8]`` tile, a team of
``64*WPR`` lanes walks the vectors with stride ``TEAM``, and the rows of a launch are dealt
to workgroups by a ``Row(workgroups, rows per workgroup)`` layout.

The arithmetic follows the reference kernels: softmax subtracts the row maximum and
divides by the sum of exponentials (softmax_sympy.py:55-80); LayerNorm computes the mean,
then the biased variance of ``x - mean`` in a second pass, ``rstd = 1/sqrt(var + eps)``,
``y = (x - mean)*rstd*w + b``, and stores ``mean`` and ``rstd`` per row
(layernorm_triton.py:101-145).  Both passes run over registers, not memory.
"""
from __future__ import annotations

from ..lego import OrderBy, Row
from .common import BANNER, Emitted, code, idx, size, template, tidy

THREADS = 256
VPTS = (1, 2, 4, 8, 16)


def emit(waves_per_row=1):
    WPR = waves_per_row
    TEAM = 64 * WPR
    RPW = THREADS // TEAM                       # rows per workgroup
    M, N, NWG = size("M"), size("N"), size("NWG")
    wg, t, it, lane, team, row, v = (idx(n) for n in ("wg", "t", "it", "lane", "team", "row", "v"))

    # thread -> (team, lane)
    team_e, lane_e = OrderBy(Row(RPW, TEAM)).TileBy([RPW, TEAM]).inv(t)
    # (workgroup, team) -> row
    rows = OrderBy(Row(NWG, RPW)).TileBy([NWG], [RPW])
    row_e = tidy(rows[wg, team], {wg: (0, NWG), team: (0, RPW)})
    # x[row][vector][8]: vector v = it*TEAM + lane of the row, as an offset in elements
    X = OrderBy(Row(M, N)).TileBy([M, N / 8], [1, 8])
    vec_e = it * TEAM + lane
    row_base = tidy(X[row, 0, 0, 0], {row: (0, M)})
    vec_off = tidy(X[0, v, 0, 0], {v: (0, N / 8)})
    stat = OrderBy(Row(M)).TileBy([M])[row,]

    params = dict(
        banner=BANNER, WPR=WPR, TEAM=TEAM, RPW=RPW, THREADS=THREADS,
        VPTS=[vp for vp in VPTS if vp * TEAM * 8 <= 65536],
        row_layout=f"OrderBy(Row(NWG, {RPW})).TileBy([NWG], [{RPW}])[wg, team]",
        lane_layout=f"OrderBy(Row({RPW}, {TEAM})).TileBy([{RPW}, {TEAM}]).inv(t); vector = it*{TEAM} + lane",
        x_layout="OrderBy(Row(M, N)).TileBy([M, N/8], [1, 8])[row, v, 0, :]",
        team=code(team_e), lane=code(lane_e), row=code(row_e),
        row_base=code(row_base).replace("row", "static_cast<size_t>(row)"),
        vec=code(vec_e), vec_off=code(vec_off), stat_off=code(stat),
    )
    text = template("rowwise.hip.j2").render(**params)
    return Emitted(f"rowwise_w{WPR}.hip", text,
                   [f"lego_softmax_f16_w{WPR}_launch", f"lego_layernorm_fwd_f16_w{WPR}_launch"])
