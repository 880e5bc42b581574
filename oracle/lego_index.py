"""TEST INFRASTRUCTURE -- CPU oracle for LEGO index maps.  Not part of the product.

Only ``tests/``, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of ``bench.py``
may import this package; nothing under ``lego_amd/`` does.

An integer-only restatement of the reference's layout semantics, evaluated eagerly on
Python ints or numpy integer arrays (no sympy, no simplification).  Each function names
the reference lines it follows:

=================  ==========================================================
``fold``           lego/lego.py:93-109   (``flatten_index``)
``unfold``         lego/lego.py:112-136  (``unflatten_index``)
``level_gather``   lego/lego.py:88-90    (``get_sigma_perm``)
``Perm``           lego/lego.py:197-228  (``RegP``; ``row``/``col`` = ``Row``/``Col`` :231-240)
``Bijection``      lego/lego.py:150-178  (``GenP``)
``Order``          lego/lego.py:288-349  (``OrderBy.apply`` / ``OrderBy.inv``)
``Layout``         lego/lego.py:388-437  (``GroupBy.apply`` / ``GroupBy.inv``)
``tile_by``        lego/lego.py:270-286  (``OrderBy.TileBy``)
=================  ==========================================================

Pinned by (see tests/test_oracle_index.py): the offset expressions the reference
committed in its generated kernels (tests/golden/reference_strings.json), the load/store
offsets of its generated transposes (tests/golden/mlir_transpose_offsets.npz), closed
forms for row/column-major tiles, and brute-force bijectivity on small extents.
"""
from __future__ import annotations

import numpy as np


def _prod(xs):
    out = 1
    for x in xs:
        out = out * x
    return out


def fold(index, extents):
    """Position of ``index`` in a row-major box of ``extents``."""
    assert len(index) == len(extents)
    pos = 0
    for i, n in zip(index, extents):
        pos = pos * n + i          # Horner form of sum(i_k * prod(n_{k+1..}))
    return pos


def unfold(pos, extents):
    """Digits of ``pos`` in the mixed radix ``extents``, most significant first."""
    digits = []
    for n in reversed(extents):
        digits.append(pos % n)
        pos = pos // n
    # the leading digit is not reduced by the reference either: pos // stride_0
    digits[-1] = digits[-1] + pos * extents[0]
    return tuple(reversed(digits))


def level_gather(rank, levels):
    return [d + rank * l for d in range(rank) for l in range(levels)]


def _take(values, perm):
    return [values[p] for p in perm]


def _invert(perm):
    out = [0] * len(perm)
    for i, p in enumerate(perm):
        out[p] = i
    return out


class Perm:
    """Regular permutation block: axis ``perm[-1]`` is the fastest in memory."""

    def __init__(self, extents, perm):
        self.extents = tuple(extents)
        self.perm = list(perm)

    def size(self):
        return _prod(self.extents)

    def apply(self, index):
        return fold(_take(index, self.perm), _take(self.extents, self.perm))

    def inv(self, pos):
        return tuple(_take(unfold(pos, _take(self.extents, self.perm)), _invert(self.perm)))


def row(*extents):
    return Perm(extents, list(range(len(extents))))


def col(*extents):
    return Perm(extents, list(range(len(extents)))[::-1])


class Bijection:
    """User bijection block (``GenP``)."""

    def __init__(self, extents, forward, backward):
        self.extents = tuple(extents)
        self.forward, self.backward = forward, backward

    def size(self):
        return _prod(self.extents)

    def apply(self, index):
        return self.forward(tuple(index))

    def inv(self, pos):
        return tuple(self.backward(pos))


class Order:
    """``OrderBy``: blocks concatenated, first block most significant."""

    def __init__(self, *blocks):
        self.blocks = blocks
        self.extents = tuple(n for b in blocks for n in b.extents)
        self.rank = len(blocks[0].extents)

    def apply(self, index):
        pos, at = 0, 0
        for b in self.blocks:
            r = len(b.extents)
            pos = pos * b.size() + b.apply(index[at:at + r])
            at += r
        return pos

    def inv(self, pos):
        parts = []
        for b in reversed(self.blocks):
            parts.insert(0, b.inv(pos % b.size()))
            pos = pos // b.size()
        return tuple(i for part in parts for i in part)


class Layout:
    """``GroupBy``: logical extents over a list of orderings.

    ``apply`` folds the logical index and pushes it through the orderings from the last
    to the first; ``inv`` pulls an offset through them from the first to the last.
    """

    def __init__(self, logical, orders):
        self.logical = tuple(logical)
        self.orders = list(orders)

    def size(self):
        return _prod(self.logical)

    def apply(self, *index):
        assert len(index) == len(self.logical)
        pos = fold(index, self.logical)
        for o in reversed(self.orders):
            pos = o.apply(unfold(pos, o.extents))
        return pos

    def inv(self, pos):
        for o in self.orders:
            pos = fold(o.inv(pos), o.extents)
        return unfold(pos, self.logical)

    def offsets(self):
        """Offset of every logical index, as an int64 array of shape ``logical``."""
        grids = np.meshgrid(*[np.arange(n, dtype=np.int64) for n in self.logical],
                            indexing="ij", sparse=True)
        return np.broadcast_to(self.apply(*grids), self.logical)


def tile_by(chain, *levels):
    """``OrderBy(...).TileBy(level0, level1, ...)`` for a chain of ``Order`` objects.

    After every ordering of the chain comes the permutation that regroups its blocks'
    extents dimension by dimension; the tiled logical index is regrouped the same way
    at the end of the list.
    """
    if isinstance(chain, Order):
        chain = [chain]
    logical = [n for level in levels for n in level]
    orders = []
    for o in chain:
        gather = level_gather(o.rank, len(o.blocks))
        orders.append(o)
        orders.append(Order(Perm(_take(list(o.extents), gather), _invert(gather))))
    orders.append(Order(Perm(logical, level_gather(len(levels[0]), len(levels)))))
    return Layout(logical, orders)


def xor_swizzle(rows, cols, unit=1, every=1, span=None):
    """Row-keyed XOR rotation of the column digit; closed form
    ``r*cols + (c ^ (((r // every) % span) * unit))``.  Not in the reference: pinned by
    bijectivity and by the bank arithmetic in tests/test_swizzle.py."""
    span = cols // unit if span is None else span

    def key(r):
        return ((r // every) % span) * unit

    return Bijection((rows, cols),
                     lambda rc: rc[0] * cols + (rc[1] ^ key(rc[0])),
                     lambda p: (p // cols, (p % cols) ^ key(p // cols)))
