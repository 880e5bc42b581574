"""Generator of the Needleman-Wunsch kernel.

The reference's contribution to this benchmark is one layout: the score tile that a block
sweeps along its anti-diagonals is stored in anti-diagonal order,
``OrderBy(GenP([n, n], antidiag)).TileBy((n, n))[i, j]``, so that the cells touched in one step
are neighbours in shared memory (benchmarks/cuda/nw_sympy.py:9-11; the Rodinia kernel around it is
benchmarks/cuda/nw/needle_kernel_temp.cu:70-160).  The recurrence is Rodinia's:
``m[i][j] = max(m[i-1][j-1] + ref[i][j], m[i][j-1] - penalty, m[i-1][j] - penalty)``.

Here a block is one 64-lane wavefront and a 64 x 64 tile: lane ``tx`` owns column ``tx`` and
walks down it one anti-diagonal behind lane ``tx - 1``, so the west and north-west neighbours
arrive by a lane shift and the north neighbour is the lane's own previous value -- the
recurrence needs no shared memory and no barrier.  What is left for LDS is a rotation: a lane
loads its column row by row, but its register slot ``k`` must hold row ``(k - tx) mod 64`` (the
row it reaches in step ``k``), and registers cannot be indexed by a lane-dependent amount.  For
that access (slot ``k`` of all lanes = one cell per column, on two anti-diagonals) a plain
``Row(64, 64)`` tile is already free of bank conflicts, lane ``tx`` always in bank ``tx``, and its
offsets are one shift and one add; the anti-diagonal order costs a ``Piecewise`` of products per
access and made the kernel 2.7 times slower (the index arithmetic was two thirds of its
instructions).  ``tile_layout()`` still builds the reference's layout; the tests pin it to the
anti-diagonal enumeration.  The offsets of the tiles of the ``(n+1) x (n+1)`` matrices are LEGO
expressions as well.
"""
from __future__ import annotations

import sympy as sp

from ..lego import GenP, OrderBy, Row, antidiag
from .common import BANNER, Emitted, code, idx, size, template, tidy

B = 64


def tile_layout(b=B):
    """The reference's anti-diagonal layout of a ``b x b`` tile."""
    return OrderBy(GenP([b, b], lambda x: antidiag(b, x), None)).TileBy((b, b))


def rotation_layout(b=B):
    """The LDS tile of the kernel: row-major, a lane's column in one bank."""
    return OrderBy(Row(b, b)).TileBy([b, b])


def emit():
    cols = size("cols")                       # n + 1: row pitch of both matrices
    by, bx, ty, tx = (idx(n) for n in ("by", "bx", "ty", "tx"))
    # cell (ty, tx) of block (by, bx); row 0 and column 0 of the matrices are the borders
    full = OrderBy(Row(cols, cols)).TileBy([cols, cols])
    cell = tidy(full[by * B + 1 + ty, bx * B + 1 + tx], {ty: (0, B), tx: (0, B)})
    # The lane's share of the offset, apart: what is left is the same for all lanes of a tile row, so
    # the accesses take a scalar base and one lane offset instead of 64-bit lane arithmetic per row.
    cell_row = tidy(cell.subs(tx, 0), {ty: (0, B)})
    cell_lane = sp.expand(cell - cell_row)
    if cell_lane.free_symbols - {tx}:
        raise ValueError(f"cell offset {cell} does not split into a row part and a lane part")
    i, j = sp.symbols("i j", integer=True, nonnegative=True)
    lds = sp.simplify(rotation_layout()[i, j])
    params = dict(
        banner=BANNER, B=B,
        tile_layout=f"OrderBy(Row({B}, {B})).TileBy([{B}, {B}])[i, j]",
        matrix_layout=f"OrderBy(Row(cols, cols)).TileBy([cols, cols])[{B}*by + 1 + ty, {B}*bx + 1 + tx]",
        cell_row=code(cell_row), cell_lane=code(cell_lane), lds=code(lds),
    )
    text = template("nw.hip.j2").render(**params)
    return Emitted("nw_i32.hip", text, ["lego_nw_i32_launch"]), dict(B=B)
