"""Generator of the LayerNorm backward kernels.

The reference computes ``dx`` per row and accumulates ``dw``/``db`` partial sums into
``GROUP_SIZE_M`` buffers of the weights' precision guarded by spin locks, then reduces those
buffers (benchmarks/triton/layernorm_triton.py:206-311, host side :352-384).  The arithmetic here
is the same -- ``xhat = (x-mean)*rstd``, ``wdy = w*dy``, ``c1 = mean(xhat*wdy)``, ``c2 = mean(wdy)``,
``dx = (wdy - (xhat*c1 + c2))*rstd``, ``dw = sum(dy*xhat)``, ``db = sum(dy)`` -- but the partial sums
stay in fp32 registers of a workgroup that walks several rows and are written once, so there
is no lock and the summation order is fixed.  The LEGO offsets are the reference's:
``N*pid + arange`` for x/dy/dx (``X_L['pid', 0, 0, :]``) and ``N*lock_id + arange`` for the
partials (``X_L['lock_id', 0, 0, :]``), with the row dealt by ``Row(steps, G)``.
"""
from __future__ import annotations

from ..lego import OrderBy, Row
from .common import BANNER, Emitted, code, idx, size, template, tidy

MAX_GROUPS = 512      # workgroups of stage 1 = rows of the partial buffers
# (lanes per row, 16-byte vectors per lane): rows of up to 2048, 4096, 8192 and 16384 elements; the
# longest rows take 512 lanes so that a lane's partial sums still fit its registers
CONFIGS = ((256, 1), (256, 2), (512, 2), (512, 4))
# Longer rows (the reference takes fp16 rows of up to 32768 elements, layernorm_triton.py:398-401):
# 1024 lanes per row leave a lane 128 registers, too few for its partial sums next to the row, so
# that kernel only writes dx, and dw/db come from a second pass over dy and x by columns.
# Rows of any length keep a few more values per lane (their head and tail elements): with four vectors per lane 256
# lanes pass 256 registers and only one workgroup stays on a CU, so rows of 4097-8192 elements take 512 lanes
# with two vectors each and the next row's loads in flight
RAGGED_CONFIGS = ((256, 1), (256, 2), (512, 2), (512, 4))
LONG = (1024, 4)
LONG_GROUPS = 64      # row slices of the column pass = rows of its partial buffers
# rows of up to WAVE_MAX_N elements: a wavefront per row (1 or 2 vectors per lane), four rows per workgroup (with 4
# vectors per lane a wave needs all 256 registers and 16384 x 2048 takes 57 us against 43)
WAVE_VS = (1, 2)
WAVE_MAX_N = 1024
WAVE_GROUPS = 1024    # workgroups of those kernels = rows of their partial buffers


ELTS = (("_Float16", "f16", "half8"), ("__bf16", "bf16", "bhalf8"), ("float", "f32", "float8v"))


def emit():
    """One translation unit per element type (they compile side by side); ``(units, constants)``."""
    return [_emit(elt) for elt in ELTS], dict(MAX_N=LONG[0] * LONG[1] * 8, MAX_GROUPS=MAX_GROUPS)


def _emit(elt):
    M, N, G, STEPS = size("M"), size("N"), size("G"), size("STEPS")
    wg, t, it, step, row, v = (idx(n) for n in ("wg", "t", "it", "step", "row", "v"))
    rows = OrderBy(Row(STEPS, G)).TileBy([STEPS], [G])
    row_e = tidy(rows[step, wg], {step: (0, STEPS), wg: (0, G)})
    X = OrderBy(Row(M, N)).TileBy([M, N / 8], [1, 8])
    P = OrderBy(Row(G, N)).TileBy([G, N / 8], [1, 8])
    params = dict(
        banner=BANNER, CONFIGS=list(CONFIGS), MAX_GROUPS=MAX_GROUPS, LONG=LONG, LONG_GROUPS=LONG_GROUPS,
        # (lanes, vectors per lane, keeps partial sums, rows of any length)
        KERNELS=[(th, v, True, False) for th, v in CONFIGS] + [(th, v, True, True) for th, v in RAGGED_CONFIGS]
        + [LONG + (False, False)],
        RAGGED_CONFIGS=list(RAGGED_CONFIGS), RAGGED_MAX_N_256=max(v for th, v in RAGGED_CONFIGS if th == 256) * 256 * 8,
        WAVE_VS=WAVE_VS, WAVE_MAX_N=WAVE_MAX_N, WAVE_GROUPS=WAVE_GROUPS,
        # every element type takes the same kernels, eight elements per lane and step: (type, tag, vector type)
        ELTS=[elt], WITH_GROUPS=elt[1] == "f16",
        MAX_N_ACC=max(th * v for th, v in CONFIGS) * 8,
        MAX_N_256=max(v for th, v in CONFIGS if th == 256) * 256 * 8,
        row_layout="OrderBy(Row(STEPS, G)).TileBy([STEPS], [G])[step, wg]",
        x_layout="OrderBy(Row(M, N)).TileBy([M, N/8], [1, 8])[row, v, 0, :]",
        part_layout="OrderBy(Row(G, N)).TileBy([G, N/8], [1, 8])[wg, v, 0, :]",
        row=code(row_e),
        row_base=code(tidy(X[row, 0, 0, 0], {row: (0, M)})).replace("row", "static_cast<size_t>(row)"),
        vecs={th: code(it * th + t) for th in sorted({64} | {th for th, _ in CONFIGS + (LONG,)})},
        vec_off=code(tidy(X[0, v, 0, 0], {v: (0, N / 8)})),
        vec_off4=code(tidy(OrderBy(Row(M, N)).TileBy([M, N / 4], [1, 4])[0, v, 0, 0], {v: (0, N / 4)})),
        stat_off=code(OrderBy(Row(M)).TileBy([M])[row,]),
        part_off=code(tidy(P[wg, v, 0, 0], {wg: (0, G), v: (0, N / 8)})).replace("wg", "static_cast<size_t>(wg)"),
    )
    text = template("layernorm_bwd.hip.j2").render(**params)
    return Emitted(f"layernorm_bwd_{elt[1]}.hip", text, [f"lego_layernorm_bwd_{elt[1]}_launch"])
