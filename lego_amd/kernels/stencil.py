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

A workgroup of 512 lanes is one brick; lane ``t`` is point ``Row(B, B, B).inv(t)`` of it, last
coordinate fastest, so a wavefront touches 64 consecutive floats of a brick (bricks storage) or
eight 32-byte runs (row-major storage).  The brick and a shell of ``radius`` points around it
are staged in LDS once; the neighbours of a point are read from there.
"""
from __future__ import annotations

from ..lego import OrderBy, Row
from .common import BANNER, Emitted, code, idx, size, template, tidy

B = 8
MAX_RADIUS = 3        # the coefficient cube is 8 x 8 x 8: offsets -3..3 plus one unused plane


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
    ijk = OrderBy(Row(B, B, B)).TileBy([B, B, B]).inv(t)
    rng = {x: (0, B * nb), y: (0, B * nb), z: (0, B * nb)}
    at = [code(tidy(L[x // B, y // B, z // B, x % B, y % B, z % B], rng)) for L in layouts(nb)]
    coeff = OrderBy(Row(8, 8, 8)).TileBy([8, 8, 8])[a, b_, c_]
    # the shell cube in LDS: row-major H x H x H, H a compile-time constant of the kernel
    H, h, hx, hy, hz = size("H"), idx("h"), idx("hx"), idx("hy"), idx("hz")
    shell = OrderBy(Row(H, H, H)).TileBy([H, H, H])
    halo_inv = [code(tidy(e, {h: (0, H * H * H)})) for e in shell.inv(h)]
    halo_at = code(tidy(shell[hx, hy, hz], {hx: (0, H), hy: (0, H), hz: (0, H)}))
    params = dict(
        banner=BANNER, B=B, MAX_RADIUS=MAX_RADIUS,
        normal_layout=f"OrderBy(Row(N, N, N)).TileBy([N/{B}]*3, [{B}]*3)[x/{B}, y/{B}, z/{B}, x%{B}, y%{B}, z%{B}]",
        bricks_layout=f"OrderBy(Row(N/{B}, N/{B}, N/{B}), Row({B}, {B}, {B})).TileBy([N/{B}]*3, [{B}]*3)[x/{B}, ...]",
        brick=[code(tidy(e, {wg: (0, nb * nb * nb)})) for e in bxyz],
        point=[code(tidy(e, {t: (0, B * B * B)})) for e in ijk],
        at_normal=at[0], at_bricks=at[1], coeff=code(coeff),
        halo_layout="OrderBy(Row(H, H, H)).TileBy([H, H, H])", halo_inv=halo_inv, halo_at=halo_at,
    )
    text = template("stencil.hip.j2").render(**params)
    return Emitted("stencil_f32.hip", text, ["lego_stencil_f32_launch"]), dict(B=B, MAX_RADIUS=MAX_RADIUS)
