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

ELEMENTS = {"f16": ("_Float16", 2), "bf16": ("__bf16", 2), "f32": ("float", 4)}
THREADS = 256                  # lanes per workgroup; a team of 16 waves is a workgroup of 1024
MAX_N = 32768                  # the reference's fp16 LayerNorm limit (64 KiB of row, layernorm_triton.py:335-338)
MAX_N_SMALL_TEAMS = 16384      # teams of up to four waves; longer rows take sixteen
LONG_ROW_WAVES = 16
VPTS = (1, 2, 4, 8, 16, 32, 64)


def emit(waves_per_row=1, dtype="f16", vectorised=True, seq_max_wpr=4, prefetch_max_wpr=4, stream_wgs=0, team_lanes=None,
         stream_min_vectors=1):
    """One translation unit: every register footprint ``V`` of one (waves per row, element type,
    access width) combination.  ``vectorised=False`` emits the kernels that take rows of any length
    and alignment (the reference's own softmax test is 1823 x 781): the elements before a row's
    first 16-byte boundary and after its last whole vector go one per lane, the rest as vectors.
    ``team_lanes`` (16 or 32) makes teams of a part of a wave for rows of at most ``team_lanes`` vectors:
    a row of 128 halves in a wave of its own would leave 48 of 64 lanes without a vector.
    ``stream_wgs`` workgroups walk the rows of a LayerNorm launch of many rows (0: no such launch), for the
    register footprints of at least ``stream_min_vectors`` vectors per lane."""
    WPR = waves_per_row
    elt, esize = ELEMENTS[dtype]
    EPV = 16 // esize
    tag = dtype if vectorised else dtype + "s"
    TEAM = 64 * WPR
    wtag = f"w{WPR}"
    if team_lanes:
        assert WPR == 1 and team_lanes in (16, 32)
        TEAM, wtag = team_lanes, f"l{team_lanes}"
    threads = max(THREADS, TEAM)
    RPW = threads // TEAM                       # rows per workgroup
    # register footprints: a lane keeps V*EPV fp32 values, at most 128; the sixteen-wave team only
    # gets the footprints that the smaller teams do not cover
    lo, hi = (MAX_N_SMALL_TEAMS, MAX_N) if WPR >= LONG_ROW_WAVES else (0, MAX_N_SMALL_TEAMS)
    M, N, NWG = size("M"), size("N"), size("NWG")
    wg, t, it, lane, team, row, v = (idx(n) for n in ("wg", "t", "it", "lane", "team", "row", "v"))

    # thread -> (team, lane)
    team_e, lane_e = OrderBy(Row(RPW, TEAM)).TileBy([RPW, TEAM]).inv(t)
    # (workgroup, team) -> row
    rows = OrderBy(Row(NWG, RPW)).TileBy([NWG], [RPW])
    row_e = tidy(rows[wg, team], {wg: (0, NWG), team: (0, RPW)})
    # x[row][vector][8]: vector v = it*TEAM + lane of the row, as an offset in elements
    X = OrderBy(Row(M, N)).TileBy([M, N / EPV], [1, EPV])
    vec_e = it * TEAM + lane
    row_base = tidy(X[row, 0, 0, 0], {row: (0, M)})
    vec_off = tidy(X[0, v, 0, 0], {v: (0, N / EPV)})
    stat = OrderBy(Row(M)).TileBy([M])[row,]
    # many rows per workgroup (LayerNorm with gamma and beta staged in LDS): workgroup wg of G walks rows
    # Row(STEPS, G)[step, wg]
    G, STEPS, step = size("G"), size("STEPS"), idx("step")
    stream_row = tidy(OrderBy(Row(STEPS, G)).TileBy([STEPS], [G])[step, wg], {step: (0, STEPS), wg: (0, G)})
    # the same walk with several teams per workgroup (rows of any length): Row(STEPS, G, RPW)[step, wg, team]
    team_rows = OrderBy(Row(STEPS, G, RPW)).TileBy([STEPS], [G], [RPW])
    stream_team_row = tidy(team_rows[step, wg, team], {step: (0, STEPS), wg: (0, G), team: (0, RPW)})
    stream_team0_row = tidy(team_rows[step, wg, 0], {step: (0, STEPS), wg: (0, G)})

    params = dict(
        banner=BANNER, WPR=WPR, TEAM=TEAM, RPW=RPW, THREADS=threads, WTAG=wtag, SHUFFLE=min(TEAM, 64),
        VPTS=[1] if team_lanes else [vp for vp in VPTS if vp * EPV <= 128 and lo < vp * TEAM * EPV <= hi],
        dtype=dtype, elt=elt, EPV=EPV, ESIZE=esize, RAGGED=not vectorised, tag=tag,
        SEQ_MAX_WPR=seq_max_wpr, PREFETCH_MAX_WPR=prefetch_max_wpr,
        STREAM=stream_wgs > 0 and (RPW == 1 or not vectorised), STREAM_WGS=stream_wgs, STREAM_MIN_V=stream_min_vectors,
        WALK_STEPS=64 if vectorised else 16,     # rows per team and launch of the walking kernels
        stream_team_layout=f"OrderBy(Row(STEPS, G, {RPW})).TileBy([STEPS], [G], [{RPW}])[step, wg, team]",
        stream_team_row=code(stream_team_row), stream_team0_row=code(stream_team0_row),
        stream_layout="OrderBy(Row(STEPS, G)).TileBy([STEPS], [G])[step, wg]", stream_row=code(stream_row),
        row_layout=f"OrderBy(Row(NWG, {RPW})).TileBy([NWG], [{RPW}])[wg, team]",
        lane_layout=f"OrderBy(Row({RPW}, {TEAM})).TileBy([{RPW}, {TEAM}]).inv(t); vector = it*{TEAM} + lane",
        x_layout=f"OrderBy(Row(M, N)).TileBy([M, N/{EPV}], [1, {EPV}])[row, v, 0, :]",
        team=code(team_e), lane=code(lane_e), row=code(row_e),
        row_base=code(row_base).replace("row", "static_cast<size_t>(row)"),
        vec=code(vec_e), vec_off=code(vec_off), stat_off=code(stat),
    )
    text = template("rowwise.hip.j2").render(**params)
    return Emitted(f"rowwise_{tag}_{wtag}.hip", text,
                   [f"lego_softmax_{tag}_{wtag}_launch", f"lego_layernorm_fwd_{tag}_{wtag}_launch"])


def emit_long():
    """Softmax of rows of any length: one workgroup of 1024 lanes per row, two passes over the row
    (a running maximum and rescaled sum, then the normalised exponentials)."""
    M, N = size("M"), size("N")
    row, v = idx("row"), idx("v")
    variants, vec_off = [], {}
    for dtype, (elt, esize) in ELEMENTS.items():
        epv = 16 // esize
        variants.append((dtype, elt, epv))
        X = OrderBy(Row(M, N)).TileBy([M, N / epv], [1, epv])
        vec_off[epv] = code(tidy(X[0, v, 0, 0], {v: (0, N / epv)}))
        row_base = tidy(X[row, 0, 0, 0], {row: (0, M)})
    text = template("softmax_long.hip.j2").render(
        banner=BANNER, THREADS=1024, VARIANTS=variants, vec_off=vec_off,
        row_base=code(row_base).replace("row", "static_cast<size_t>(row)"),
        x_layout="OrderBy(Row(M, N)).TileBy([M, N/EPV], [1, EPV])[row, v, 0, :]")
    return Emitted("softmax_long.hip", text, [f"lego_softmax_long_{d}_launch" for d in ELEMENTS])
