"""Generator of the vectorised, LDS-staged transpose.

The reference states a transpose as "copy every logical index from a row-major tiled
layout to the column-major layout with the same tiling", decoding the block id row-major
for reads and column-major for writes so that both sides are contiguous
(benchmarks/mlir/transpose_smem.py:28-80).  This generator keeps that statement -- the
source, destination and staging tiles are LEGO layouts and every address in the kernel is
printed from them -- and changes what a lane moves: one 16-byte vector per access instead
of one element, through a staging tile that is stored transposed with an XOR rotation
instead of the reference's conflicting 32x32 array.

Layouts (``R x C`` matrix, LEGO tiles ``TR x TC``, a workgroup owns ``MR x MC`` tiles):

* source       ``OrderBy(Row(R, C)).TileBy([R/SR, C/SC], [MR, MC], [TR, TC])``
* destination  ``OrderBy(Col(R, C)).TileBy(...same levels...)``
* staging      ``OrderBy(GenP((KD, SR), swizzle)).TileBy([KD, SR])`` in 4-byte words, where
  word-column ``k`` of row ``r`` holds source columns ``k`` (fp32) or ``2k, 2k+1`` (fp16).
"""
from __future__ import annotations

import sympy as sp

from ..lego import BitXor, Col, GenP, OrderBy, Row  # noqa: F401
from .common import BANNER, Emitted, code, idx, size, template, tidy

THREADS = 256
FEW_RESIDENT_FROM = 4096     # macro tiles of a launch from which three resident workgroups per CU are ahead of four or five


def lane_block(esize):
    """Rows x vectors that the 64 lanes of one wave instruction cover in phase 1.

    A lane scatters the four words of its vector into four word-columns at the same row
    digit.  The LDS serves 4-byte accesses 32 lanes at a time over 32 banks, so the 32 lanes
    of a pass must differ in ``address % 32``: four rows (bits 0-1, below the XOR key) times
    eight vectors (spread by the key over bits 2-4); the other four rows form the second pass.
    """
    return (8, 8)


def pack_factor(sr):
    """Word-columns packed into one LDS row so that a row spans all 64 banks."""
    return max(1, 64 // sr)


def staging_key(k, sr, esize):
    """XOR key of word-column ``k``; a multiple of 4, so 16-byte row groups stay whole.

    ``4*((k//4) % 8)`` sends the eight vectors of a phase-1 pass to different groups of four
    banks (the four rows of the pass fill a group); for fp16 ``4*(k%2)`` additionally separates the two
    word-columns that share a 16-lane group of 16-byte reads in phase 2.  With a packed row
    (``sr < 64``) the key only depends on ``k // pack_factor``, which keeps the map a
    bijection of the row.
    """
    lr, lc = lane_block(esize)
    key = ((k // 4) % lc) * 4
    return key if esize == 4 else _xor(key, (k % 2) * 4)


def _xor(a, b):
    if isinstance(a, sp.Expr) or isinstance(b, sp.Expr):
        return BitXor(sp.sympify(a), sp.sympify(b))
    return a ^ b


def staging_word(k, r, sr, esize):
    """Word address of (word-column ``k``, row ``r``) in the staging tile."""
    p = pack_factor(sr)
    return (k // p) * (p * sr) + _xor((k % p) * sr + r, staging_key(k, sr, esize))


def staging_layout(kd, sr, esize):
    """The staging tile as a LEGO layout: ``OrderBy(GenP((kd, sr), xor-rotated rows)).TileBy([kd, sr])``."""
    p = pack_factor(sr)

    def backward(flat):
        j, pos = flat // (p * sr), flat % (p * sr)
        raw = _xor(pos, staging_key(j * p, sr, esize))   # the key is the same for every k of row j
        return (j * p + raw // sr, raw % sr)

    return OrderBy(GenP((kd, sr), lambda kr: staging_word(kr[0], kr[1], sr, esize), backward)).TileBy([kd, sr])


def phase1_vector(sr, w, esize, it, t):
    """``(row, vector)`` that lane ``t`` of a 256-lane workgroup loads in step ``it`` of phase 1.

    The vectors of the macro tile form an ``[sr, w]`` box tiled by the lane block; a wave
    instruction covers one block and the four waves of a step take adjacent column blocks, so
    a step reads ``LR`` row segments of up to ``4*LC`` contiguous vectors.  Works on ints (the
    bank-arithmetic test) and on symbols (the generator).
    """
    lr, lc = lane_block(esize)
    assert sr % lr == 0 and w % lc == 0
    symbolic = isinstance(it, sp.Expr) or isinstance(t, sp.Expr)
    inv = (lambda lay, x: lay.inv(x)) if symbolic else (lambda lay, x: lay.inv_raw(x))
    blocks = OrderBy(Row(sr // lr, w // lc)).TileBy([sr // lr, w // lc])
    lanes = OrderBy(Row(lr, lc)).TileBy([lr, lc])
    vectors = OrderBy(Row(sr, w)).TileBy([sr // lr, w // lc], [lr, lc])
    rb, cb = inv(blocks, it * (THREADS // 64) + t // 64)
    dr, cvl = inv(lanes, t % 64)
    flat = vectors[rb, cb, dr, cvl] if symbolic else vectors.apply(rb, cb, dr, cvl)
    return inv(OrderBy(Row(sr, w)).TileBy([sr, w]), flat)


def tile_order(order, n_bi, n_bj, wg):
    """Workgroup id -> macro tile ``(Bi, Bj)``.

    ``row``: tiles of one tile-row are consecutive (contiguous reads, strided writes);
    ``col``: the transpose of that (strided reads, contiguous writes);
    ``diag``: row order skewed by the tile row, ``Bj = (j + Bi) % n_bj``, so that workgroups
    that run together spread both their reads and their writes over tile columns -- the
    classic remedy for DRAM channel camping when the row pitch is a power of two;
    ``("window", ti, tj)``: row order inside windows of ``ti x tj`` tiles, windows in row
    order; ``n_bi`` and ``n_bj`` must be multiples of ``ti`` and ``tj``;
    ``("strip", w)``: row order inside strips of ``w`` tile columns, any ``n_bi`` and ``n_bj``.
    """
    if order == "row":
        return OrderBy(Row(n_bi, n_bj)).TileBy([n_bi, n_bj]).inv(wg)
    if order == "col":
        return OrderBy(Col(n_bi, n_bj)).TileBy([n_bi, n_bj]).inv(wg)
    if order == "diag":
        skew = GenP((n_bi, n_bj),
                    lambda ij: ij[0] * n_bj + (ij[1] - ij[0]) % n_bj,
                    lambda f: (f // n_bj, (f % n_bj + f // n_bj) % n_bj))
        return OrderBy(skew).TileBy([n_bi, n_bj]).inv(wg)
    if isinstance(order, tuple) and order[0] == "window":
        # windows of ti x tj tiles, row-major inside and across: with a window about as large
        # as the set of workgroups in flight, the reads of that set are tj tiles wide per row
        # and its writes ti tiles wide per output row, so both sides keep DRAM pages open
        _, ti, tj = order
        windows = OrderBy(Row(n_bi / ti, n_bj / tj), Row(ti, tj)).TileBy([n_bi / ti, n_bj / tj], [ti, tj])
        wi, wj, i, j = windows.inv(wg)
        return wi * ti + i, wj * tj + j
    if isinstance(order, tuple) and order[0] == "strip":
        # strips of w tile columns (the last one narrower), row order inside a strip: the workgroups in flight cover
        # a block of tiles some w wide and as many rows deep as fit, so that a tile's neighbours on all four sides
        # run with it -- for shapes whose tile edges cut 128-byte lines in both matrices
        _, w = order
        if isinstance(wg, sp.Expr):
            strip = sp.Min(sp.floor(wg / (n_bi * w)), sp.floor(n_bj / w))
            width = sp.Min(w, n_bj - strip * w)
            rem = wg - strip * n_bi * w
            return sp.floor(rem / width), strip * w + sp.Mod(rem, width)
        strip = min(wg // (n_bi * w), n_bj // w)
        width = min(w, n_bj - strip * w)
        rem = wg - strip * n_bi * w
        return rem // width, strip * w + rem % width
    raise ValueError(order)


def emit(dtype="f32", tile=(32, 32), group=(2, 2), order="row", suffix="", edge=False, ragged=False, xcd=False,
         stream_loads=False):
    """HIP translation unit for one element type and one tiling.  ``edge``: the shape need not be
    a whole number of macro tiles, only of 16-byte vectors in both directions; vectors past the
    edge are skipped.  ``ragged`` (with ``edge``): any shape; rows start at any element, the vectors
    that an edge cuts go element by element.  ``xcd`` (with ``edge``): workgroup ids are dealt to the tiles
    so that each XCD takes a contiguous run of them (``order`` is then the order inside that run).
    ``stream_loads`` (with ``edge``): non-temporal loads, as the kernels for whole tiles use; without it the 128-byte
    lines that the row segments of neighbouring tiles share stay in the L2 for the neighbour."""
    elt, esize = {"f32": ("float", 4), "f16": ("_Float16", 2)}[dtype]
    vec = 16 // esize                       # elements per 16-byte vector
    (TR, TC), (MR, MC) = tile, group
    SR, SC = MR * TR, MC * TC               # macro tile of a workgroup, in elements
    KD = SC * esize // 4                    # word-columns of the staging tile
    rows_per_read = 16 // 4 if esize == 4 else 8
    assert (SR * SC) % (vec * THREADS) == 0 and SR % rows_per_read == 0
    P1 = SR * SC // (vec * THREADS)
    P2 = KD * (SR // rows_per_read) // THREADS
    assert P2 >= 1 and KD * (SR // rows_per_read) % THREADS == 0

    R, C = size("R"), size("C")
    wg, t, it, e = idx("wg"), idx("t"), idx("it"), idx("e")
    r, cv, k, rv = idx("r"), idx("cv"), idx("k"), idx("rv")
    Bi, Bj = idx("Bi"), idx("Bj")
    levels = ([R / SR, C / SC], [MR, MC], [TR, TC])
    src = OrderBy(Row(R, C)).TileBy(*levels)
    dst = OrderBy(Col(R, C)).TileBy(*levels)
    lds = staging_layout(KD, SR, esize)

    def in_tile(layout, row, col, ranges):
        off = layout[Bi, Bj, row // TR, col // TC, row % TR, col % TC]
        return tidy(off, ranges)

    # workgroup -> macro tile, row-major over the grid of macro tiles
    nBi, nBj = size("nBi"), size("nBj")
    windowed = isinstance(order, tuple) and order[0] == "window"
    if windowed:
        # tile counts as multiples of the window, so that every division is exact
        WI, WJ = order[1:]
        Bi_e, Bj_e = tile_order(order, WI * size("nWi"), WJ * size("nWj"), wg)
        Bi_e, Bj_e = tidy(Bi_e, {}), tidy(Bj_e, {})
        suffix = f"_w{WI}x{WJ}{suffix}"
    else:
        WI = WJ = 1
        Bi_e, Bj_e = tile_order(order, nBi, nBj, wg)
    # lane -> vector of the macro tile, phase 1
    W = SC // vec
    v1 = [tidy(x, {t: (0, THREADS), it: (0, P1)}) for x in phase1_vector(SR, W, esize, it, t)]
    # lane -> (word-column, row group), phase 2
    v2 = OrderBy(Row(KD, SR // rows_per_read)).TileBy([KD, SR // rows_per_read]).inv(it * THREADS + t)
    v2 = [tidy(x, {t: (0, THREADS), it: (0, P2)}) for x in v2]

    if edge:
        assert not windowed
        suffix = f"{suffix}_ragged" if ragged else f"{suffix}_edge"
    assert edge or not (ragged or xcd)
    rng1 = {r: (0, SR), cv: (0, SC // vec), e: (0, 4)}
    rng2 = {k: (0, KD), rv: (0, SR // rows_per_read)}
    cols_per_word = 4 // esize
    params = dict(
        banner=BANNER, elt=elt, esize=esize, SR=SR, SC=SC, KD=KD, THREADS=THREADS, P1=P1, P2=P2,
        kernel=f"lego_transpose_{dtype}_{SR}x{SC}{suffix}",
        src_layout=f"OrderBy(Row(R, C)).TileBy([R/{SR}, C/{SC}], [{MR}, {MC}], [{TR}, {TC}])",
        dst_layout=f"OrderBy(Col(R, C)).TileBy([R/{SR}, C/{SC}], [{MR}, {MC}], [{TR}, {TC}])",
        lds_layout=f"OrderBy(GenP(({KD}, {SR}), xor-rotated rows)).TileBy([{KD}, {SR}])",
        Bi=code(Bi_e), Bj=code(Bj_e), WI=WI, WJ=WJ, windowed=windowed,
        p1_r=code(v1[0]), p1_cv=code(v1[1]),
        src_off=code(in_tile(src, r, cv * vec, rng1)),
        lds_store=code(tidy(lds[cv * 4 + e, r], rng1)),
        p2_k=code(v2[0]), p2_rv=code(v2[1]),
        lds_load0=code(tidy(lds[k, rv * rows_per_read], rng2)),
        lds_load1=code(tidy(lds[k, rv * rows_per_read + 4], rng2)) if esize == 2 else "",
        dst_off0=code(in_tile(dst, rv * rows_per_read, k * cols_per_word, rng2)),
        dst_off1=code(in_tile(dst, rv * rows_per_read, k * cols_per_word + 1, rng2)) if esize == 2 else "",
        xcd=xcd,
        # whole-tile kernels: from FEW_FROM macro tiles on, an LDS footprint that leaves three workgroups on a CU
        FEW_FROM=FEW_RESIDENT_FROM, FEW_LDS_BYTES=163840 // 3 // 1024 * 1024,
        grid=(f"(static_cast<unsigned>((rows + {SR - 1}) / {SR}) * static_cast<unsigned>((cols + {SC - 1}) / {SC}) + 7) / 8 * 8" if edge and xcd else
              f"static_cast<unsigned>((rows + {SR - 1}) / {SR}) * static_cast<unsigned>((cols + {SC - 1}) / {SC})" if edge
              else f"static_cast<unsigned>(rows / {SR}) * static_cast<unsigned>(cols / {SC})"),
        edge=edge, ragged=ragged, stream_loads=stream_loads, VEC=vec, bits_t="uint32_t" if esize == 4 else "uint16_t",
        # matrix coordinates of the vectors, for the edge tests: source (row, first column) in phase 1,
        # destination (row = source column, first column = source row) in phase 2
        p1_row=code(tidy(OrderBy(Row(nBi, SR)).TileBy([nBi], [SR])[Bi, r], {r: (0, SR)})),
        p1_col=code(tidy(OrderBy(Row(nBj, SC // vec, vec)).TileBy([nBj], [SC // vec], [vec])[Bj, cv, 0], {cv: (0, SC // vec)})),
        p2_row0=code(tidy(OrderBy(Row(nBj, KD, cols_per_word)).TileBy([nBj], [KD], [cols_per_word])[Bj, k, 0], {k: (0, KD)})),
        p2_col=code(tidy(OrderBy(Row(nBi, SR // rows_per_read, rows_per_read)).TileBy([nBi], [SR // rows_per_read], [rows_per_read])[Bi, rv, 0],
                         {rv: (0, SR // rows_per_read)})),
    )
    text = template("transpose.hip.j2").render(**params)
    return Emitted(f"transpose_{dtype}{suffix}.hip", text, [params["kernel"] + "_launch"]), dict(
        SR=SR, SC=SC, kernel=params["kernel"], row_multiple=SR * WI, col_multiple=SC * WJ)


def emit_any():
    """The one-element-per-access fallback for shapes that no vectorised tiling divides: the
    reference's row-major source and column-major destination with run-time sizes."""
    R, C = size("R"), size("C")
    r, c, t = idx("r"), idx("c"), idx("t")
    src = OrderBy(Row(R, C)).TileBy([R, C])
    dst = OrderBy(Col(R, C)).TileBy([R, C])
    ty_e, tx_e = OrderBy(Row(4, 64)).TileBy([4, 64]).inv(t)
    rng = {r: (0, R), c: (0, C)}
    params = dict(banner=BANNER, src_layout="OrderBy(Row(R, C)).TileBy([R, C])[r, c]",
                  dst_layout="OrderBy(Col(R, C)).TileBy([R, C])[r, c]",
                  src_off=code(tidy(src[r, c], rng)), dst_off=code(tidy(dst[r, c], rng)),
                  tx=code(tidy(tx_e, {t: (0, 256)})), ty=code(tidy(ty_e, {t: (0, 256)})))
    text = template("transpose_any.hip.j2").render(**params)
    return Emitted("transpose_any.hip", text, ["lego_transpose_any_launch"])


def python_offsets(tile_r, tile_c):
    """The transpose as the reference's Python/Triton backend states it: the printed offsets of logical
    index ``(bi, bj, i, j)`` in the row-major source ``OrderBy(Row(R, C)).TileBy([R/TR, C/TC], [TR, TC])``
    and in the column-major destination with the same tiling, every index a whole axis
    (``tl.arange(...)`` broadcast along its own axis of a rank-4 block).  Evaluated with
    ``torch.arange`` standing for ``tl.arange`` this text is LEGO's CPU index path
    (lego/lego_python.py:5-37); ``nbi`` and ``nbj`` are the numbers of tile rows and columns taken."""
    from ..lego import TritonRange, get_arange
    from ..lego_python import LEGOPythonCodePrinter
    R, C, nbi, nbj = size("R"), size("C"), size("nbi"), size("nbj")
    axes = [TritonRange(get_arange(0, n), a, 4) for a, n in enumerate((nbi, nbj, tile_r, tile_c))]
    levels = ([R / tile_r, C / tile_c], [tile_r, tile_c])
    printer = LEGOPythonCodePrinter(allow_unknown_functions=True)
    src = OrderBy(Row(R, C)).TileBy(*levels)[tuple(axes)]
    dst = OrderBy(Col(R, C)).TileBy(*levels)[tuple(axes)]
    return printer.doprint(sp.simplify(src)), printer.doprint(sp.simplify(dst))
