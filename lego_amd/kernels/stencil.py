"""Generator of the 3-D stencil kernels on row-major and on "bricks" storage.

The reference's two stencil benchmarks compare a row-major ``N^3`` array,
``OrderBy(Row(N, N, N)).TileBy([N/B]*3, [B]*3)``, with the same array stored as contiguous
``B^3`` bricks, ``OrderBy(Row(N/B, N/B, N/B), Row(B, B, B)).TileBy([N/B]*3, [B]*3)``, ``B = 8``
(benchmarks/cuda/bricks_f3d.py:8-22, bricks_laplasian.py:8-33); a thread block is a brick, and
points closer than ``radius`` to the boundary are left untouched:

* ``f3d``        ``out = in*c[r,r,r] + sum_{|di|,|dj|,|dk| <= r} in[+di,+dj,+dk] * c[di+r, dj+r, dk+r]``
  with ``c`` an ``8 x 8 x 8`` array (benchmarks/cuda/bricks/main_tmp.cu:24-66);
* ``laplacian``  ``out = in*c[0] + sum_{a=1..r} c[a] * (six neighbours at distance a)``
  (benchmarks/cuda/bricks-laplace/main_tmp.cu:24-57).

The reference indexes a neighbour as ``L[bx, by, bz, i+di, j+dj, k+dk]``, and its simplifier, told
that every index is in range, prints ``... + 64*i + 64*i_diff + ...`` for the bricks layout
(benchmarks/cuda/bricks/main.cu:99): a neighbour across a brick face is then taken from the wrong
brick.  Here a neighbour is addressed by its global coordinates, ``L[x/B, y/B, z/B, x%B, y%B, z%B]``,
so both storage orders give the stencil's result.

A wavefront is one brick; lane ``l`` owns row ``Row(B, B).inv(l)`` of it, the ``B`` points along the
last axis: 32 contiguous bytes in both storage orders, kept in registers.  A wavefront's access
to one row of every lane is the whole 2 KiB brick (bricks storage) or 64 runs of 32 bytes
(row-major storage).  The neighbours along the last axis are the lane's own registers plus
``radius`` points on either side; the other neighbours are whole rows again, fetched the same way.
"""
from __future__ import annotations

from ..lego import OrderBy, Row
from .common import BANNER, Emitted, code, idx, size, template, tidy

B = 8
MAX_RADIUS = 3        # the coefficient cube is 8 x 8 x 8: offsets -3..3 plus one unused plane
STAR_MAX_RADIUS = 4   # the star stencil has radius + 1 coefficients; the reference runs it up to 4 (result/cuda/bricks-laplace.txt)
WAVES = 4             # bricks per workgroup, dense stencil (its shell fills the 64 KiB of LDS at radius 3)
STAR_WAVES = 8        # and star stencil: the more bricks in a row, the fewer row ends come from memory
# words per row of the shell in LDS: 16 hold a row (3 + 8 + 3 points, 16-byte aligned), 20 spread the
# 16-byte reads of eight neighbouring lanes over different banks
ROW_WORDS = 20


UNPADDED_RADIUS = 2    # its padding would cost the third workgroup per CU, which is worth more (measured)


def shell_plane(radius):
    """Words between the planes ``hx`` of the shell in LDS.  A 16-byte access of 64 lanes is served 16
    lanes at a time, rows ``(i, 0..7)`` and ``(i+1, 0..7)`` of the shell: with rows ``ROW_WORDS`` = 20
    words apart the eight rows of one plane start in eight different groups of four banks
    (``5*j mod 16``), and the padding puts the next plane eight groups further, on the other eight."""
    h, g = B + 2 * radius, ROW_WORDS // 4
    pad = 0 if radius == UNPADDED_RADIUS else 4 * ((8 - g * h) % 16)
    return h * ROW_WORDS + pad


def layouts(nb):
    """``(row-major, bricks)`` layouts of a cube of ``nb`` bricks per side."""
    levels = ([nb, nb, nb], [B, B, B])
    return (OrderBy(Row(B * nb, B * nb, B * nb)).TileBy(*levels),
            OrderBy(Row(nb, nb, nb), Row(B, B, B)).TileBy(*levels))


def emit():
    nb = size("nb")
    wg, t = idx("wg"), idx("t")
    x, y, z = idx("x"), idx("y"), idx("z")
    a, b_, c_ = idx("ca"), idx("cb"), idx("cc")
    bxyz = OrderBy(Row(nb, nb, nb)).TileBy([nb, nb, nb]).inv(wg)
    ij = OrderBy(Row(B, B)).TileBy([B, B]).inv(t)
    rng = {x: (0, B * nb), y: (0, B * nb), z: (0, B * nb)}
    at = [code(tidy(L[x // B, y // B, z // B, x % B, y % B, z % B], rng)) for L in layouts(nb)]
    coeff = OrderBy(Row(8, 8, 8)).TileBy([8, 8, 8])[a, b_, c_]
    # the rows of a brick and its shell in LDS: H x H rows of ROW_WORDS words, H a compile-time constant
    H, h, hx, hy = size("H"), idx("h"), idx("hx"), idx("hy")
    shell_rows = OrderBy(Row(H, H)).TileBy([H, H])
    shell_inv = [code(tidy(e, {h: (0, H * H)})) for e in shell_rows.inv(h)]
    # rows hy of one hx are ROW_WORDS apart, the planes hx are PLANE >= H*ROW_WORDS words apart (padded so that
    # the sixteen lanes of one 16-byte access, rows (i, 0..7) and (i+1, 0..7), fall into sixteen different
    # groups of four banks: see the kernel source)
    PLANE = size("PLANE")
    shell = OrderBy(Row(H, PLANE)).TileBy([H, PLANE])
    shell_row = code(tidy(shell[hx, ROW_WORDS * hy], {hx: (0, H), hy: (0, H)}))
    # the star stencil exchanges only the B points of a row: planes of B*H + 4 words
    SPLANE = size("PLANE")
    star = OrderBy(Row(H, SPLANE)).TileBy([H, SPLANE])
    star_row = code(tidy(star[hx, B * hy], {hx: (0, H), hy: (0, H)}))
    params = dict(
        star_layout=f"OrderBy(Row(H, PLANE)).TileBy([H, PLANE])[hx, {B}*hy + word]", star_row=star_row,
        shell_layout=f"OrderBy(Row(H, PLANE)).TileBy([H, PLANE])[hx, {ROW_WORDS}*hy + word]",
        shell_inv=shell_inv, shell_row=shell_row, ROW_WORDS=ROW_WORDS,
        PLANES={B + 2 * r: shell_plane(r) for r in range(1, MAX_RADIUS + 1)},
        banner=BANNER, B=B, MAX_RADIUS=MAX_RADIUS, STAR_MAX_RADIUS=STAR_MAX_RADIUS, WAVES=WAVES, STAR_WAVES=STAR_WAVES,
        row_layout=f"Row({B}, {B})",
        normal_layout=f"OrderBy(Row(N, N, N)).TileBy([N/{B}]*3, [{B}]*3)[x/{B}, y/{B}, z/{B}, x%{B}, y%{B}, z%{B}]",
        bricks_layout=f"OrderBy(Row(N/{B}, N/{B}, N/{B}), Row({B}, {B}, {B})).TileBy([N/{B}]*3, [{B}]*3)[x/{B}, ...]",
        brick=[code(tidy(e, {wg: (0, nb * nb * nb)})) for e in bxyz],
        row=[code(tidy(e, {t: (0, B * B)})) for e in ij],
        at_normal=at[0], at_bricks=at[1], coeff=code(coeff),
    )
    text = template("stencil.hip.j2").render(**params)
    return Emitted("stencil_f32.hip", text, ["lego_stencil_f32_launch"]), dict(B=B, MAX_RADIUS=MAX_RADIUS, STAR_MAX_RADIUS=STAR_MAX_RADIUS)
