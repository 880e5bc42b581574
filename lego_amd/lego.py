"""LEGO layout algebra: bijections between logical index spaces and flat offsets.

This is the front end every lowering shares.  It keeps the names, call surface
and semantics of the reference's layout module (reference: lego/lego.py) so that
generator scripts written against it run unchanged:

``Row``/``Col``/``RegP``/``GenP``
    permutation blocks over a list of extents (lego/lego.py:150-240);
``OrderBy``
    concatenation of permutation blocks, most significant first (:243-362);
``GroupBy`` / ``OrderBy.TileBy``
    a logical (tiled) view on top of a chain of ``OrderBy`` levels; ``layout[...]``
    gives the simplified flat offset of a logical index, ``layout.inv(flat)`` the
    simplified logical index of an offset (:365-487).

Indices may be Python ints, numpy integer arrays or sympy expressions: the maps
only use ``+ * // %``.  Simplification of symbolic results is delegated to
``lego_amd.simplifier.simplify_ops``, which needs no SMT solver.
"""
from __future__ import annotations

import math
from functools import reduce
from typing import Callable, List, Sequence, Tuple

import sympy as sp
from sympy import Function, Piecewise, Symbol, symbols  # re-exported, as generator scripts expect

from .simplifier import BitXor, simplify_ops

__all__ = [
    "TritonRange", "get_arange", "product", "divisibility_constraint", "le_constraint",
    "equal_constraint", "get_sigma_perm", "flatten_index", "unflatten_index", "LayoutBlock",
    "GenP", "sigma", "inverse_permutation", "RegP", "Row", "Col", "OrderBy", "GroupBy",
    "antidiag", "antidiag_inv", "new_antidiag", "BitXor", "xor_swizzle", "XorSwizzle",
    "sp", "Symbol", "symbols", "Piecewise", "Function", "List", "Tuple", "Callable",
]


# ---------------------------------------------------------------------------
# index vectors
# ---------------------------------------------------------------------------

class TritonRange(Function):
    """A whole axis of indices used as one operand.

    ``TritonRange(vec, axis, rank)`` stands for the index vector ``vec`` (normally
    ``tl.arange(lo, hi)``) laid along ``axis`` of a rank-``rank`` block of lanes
    (reference: lego/lego.py:10-64).  It is integer valued and never evaluated; each
    printer decides what a lane vector is in its target (a broadcast slice for
    Python/Triton, a per-lane scalar for HIP).
    """

    nargs = 3
    is_integer = True
    is_nonnegative = True

    @classmethod
    def eval(cls, vec, axis, rank):
        return None

    def broadcast_suffix(self):
        axis, rank = self.args[1], self.args[2]
        if axis.is_Integer and rank.is_Integer:
            return ", ".join(":" if i == int(axis) else "None" for i in range(int(rank)))
        return f"None at dim {axis} and ':' otherwise"

    def _sympystr(self, printer):
        return f"(({printer.doprint(self.args[0])})[{self.broadcast_suffix()}])"


def get_arange(start, stop):
    """``tl.arange(start, stop)`` as an opaque integer-valued sympy application."""
    return Function("tl.arange", integer=True)(start, stop)


def product(values: Sequence):
    return reduce(lambda acc, v: acc * v, values)


def divisibility_constraint(lhs, rhs):
    return sp.Eq(lhs % rhs, 0, evaluate=False)


def le_constraint(lhs, rhs):
    return sp.StrictLessThan(lhs, rhs, evaluate=False)


def equal_constraint(lhs, rhs):
    return sp.Eq(lhs, rhs, evaluate=False)


# ---------------------------------------------------------------------------
# mixed radix arithmetic and small permutations
# ---------------------------------------------------------------------------

def get_sigma_perm(d: int, q: int) -> List[int]:
    """Positions that gather ``q`` levels of rank ``d`` dimension by dimension.

    A tiled index is stored level by level, ``(l0d0, l0d1, .., l1d0, l1d1, ..)``;
    the permutation lists, for each dimension in turn, its entry on every level:
    ``[0, d, 2d, .., 1, d+1, ..]`` (reference: lego/lego.py:88-90).
    """
    return [dim + d * level for dim in range(d) for level in range(q)]


def _strides(dims: Sequence):
    """Row-major strides of ``dims``: ``stride[k] = prod(dims[k+1:])``."""
    out = [1] * len(dims)
    for k in range(len(dims) - 2, -1, -1):
        out[k] = out[k + 1] * dims[k + 1]
    return out


def flatten_index(indices: Sequence, dims: Sequence):
    """``sum(i_k * prod(n_{k+1..}))`` -- the row-major position of ``indices`` in ``dims``
    (reference: lego/lego.py:93-109)."""
    if len(indices) != len(dims):
        raise ValueError("Number of indices must match number of dimensions")
    flat = 0
    for i, s in zip(indices, _strides(dims)):
        flat = flat + i * s
    return flat


def unflatten_index(flat_index, dims: Sequence) -> tuple:
    """Digits of ``flat_index`` in the mixed radix ``dims`` (reference: lego/lego.py:112-136)."""
    digits = []
    rest = flat_index
    for s in _strides(dims):
        digits.append(rest // s)
        rest = rest % s
    return tuple(digits)


def sigma(values: Sequence, permutation: Sequence[int]) -> list:
    """``out[i] = values[permutation[i]]`` (reference: lego/lego.py:181-186)."""
    return [values[p] for p in permutation]


def inverse_permutation(p: Sequence[int]) -> List[int]:
    inv = [0] * len(p)
    for position, target in enumerate(p):
        inv[target] = position
    return inv


# ---------------------------------------------------------------------------
# permutation blocks
# ---------------------------------------------------------------------------

class LayoutBlock:
    """Anything with ``apply(index tuple) -> flat``, ``inv(flat) -> index tuple`` and ``dims()``."""

    def apply(self, idx):
        raise NotImplementedError

    def inv(self, flat_idx):
        raise NotImplementedError

    def dims(self):
        raise NotImplementedError


class GenP(LayoutBlock):
    """A user-supplied bijection of ``nd`` onto ``[0, prod(nd))`` (reference: lego/lego.py:150-178)."""

    def __init__(self, nd, f_apply, f_inv):
        self._dims = nd
        self.f_apply = f_apply
        self.f_inv = f_inv

    def apply(self, idx):
        if len(idx) != len(self._dims):
            raise ValueError("Input index dimension mismatch")
        return self.f_apply(idx)

    def inv(self, flat_idx):
        return self.f_inv(flat_idx)

    def dims(self):
        return self._dims


class RegP(LayoutBlock):
    """Dimension permutation: store ``nd`` with axis ``perm[0]`` slowest, ``perm[-1]`` fastest
    (reference: lego/lego.py:197-228)."""

    def __init__(self, nd, perm):
        self._dims = nd
        self._perm = list(perm)
        self._perm_inv = inverse_permutation(self._perm)
        # kept as attributes for scripts that poke at them
        self.perm = lambda idx: sigma(idx, self._perm)
        self.perm_inv = lambda idx: sigma(idx, self._perm_inv)

    def apply(self, idx):
        if len(idx) != len(self._dims):
            raise ValueError("Input index dimension mismatch")
        return flatten_index(sigma(idx, self._perm), sigma(self._dims, self._perm))

    def inv(self, flat_idx):
        stored = unflatten_index(flat_idx, sigma(self._dims, self._perm))
        return sigma(stored, self._perm_inv)

    def dims(self):
        return self._dims


def Row(*group_dims):
    """Row-major order: last dimension fastest."""
    return RegP(group_dims, list(range(len(group_dims))))


def Col(*group_dims):
    """Column-major order: first dimension fastest."""
    return RegP(group_dims, list(range(len(group_dims)))[::-1])


# ---------------------------------------------------------------------------
# OrderBy / GroupBy
# ---------------------------------------------------------------------------

class OrderBy(LayoutBlock):
    """Concatenated permutation blocks; the first block is the most significant digit
    (reference: lego/lego.py:243-362)."""

    def __init__(self, *perms: LayoutBlock):
        self.perms = perms
        self._cached_dims = tuple(d for p in perms for d in p.dims())
        self.q = len(perms)
        self.d = len(perms[0].dims())
        self.chain = [self]

    # chaining ---------------------------------------------------------------
    def OrderBy(self, *perms: LayoutBlock):
        nxt = OrderBy(*perms)
        nxt.chain = self.chain + [nxt]
        self.chain.append(nxt)
        return self

    def GroupBy(self, group_dims, user_constraints=[]):
        return GroupBy(group_dims, self.chain, user_constraints)

    def TileBy(self, *group_dims, user_constraints=[]):
        """Tiled logical view ``(level0 dims.., level1 dims.., ..)`` of this physical order.

        Each ``OrderBy`` level of the chain is followed by the regular permutation that
        regroups its per-block dimensions dimension by dimension, and the chain ends with
        the permutation that does the same to the tiled logical index, so that a logical
        ``(tile.., element..)`` index lands on the right physical digit
        (reference: lego/lego.py:270-286).
        """
        logical = tuple(d for level in group_dims for d in level)
        rank, levels = len(group_dims[0]), len(group_dims)
        objects = []
        for o in self.chain:
            block_dims = [d for p in o.perms for d in p.dims()]
            gather = get_sigma_perm(o.d, o.q)
            objects.append(o)
            objects.append(OrderBy(RegP(sigma(block_dims, gather), inverse_permutation(gather))))
        objects.append(OrderBy(RegP(logical, get_sigma_perm(rank, levels))))
        return GroupBy([logical], objects, user_constraints)

    # maps -------------------------------------------------------------------
    def apply(self, idx):
        if len(idx) != len(self._cached_dims):
            raise ValueError(
                f"Input index length {len(idx)} must match combined dimension length "
                f"{len(self._cached_dims)}")
        flat, at = 0, 0
        for p in self.perms:
            n = len(p.dims())
            flat = flat * product(p.dims()) + p.apply(idx[at:at + n])
            at += n
        return flat

    def inv(self, flat_idx):
        pieces = []
        rest = flat_idx
        for p in reversed(self.perms):
            size = product(p.dims())
            if size == 0:
                raise ValueError("Permutation dimensions cannot be zero")
            pieces.append(list(p.inv(rest % size)))
            rest = rest // size
        return tuple(i for piece in reversed(pieces) for i in piece)

    def dims(self):
        return self._cached_dims


def _fewer_ops(*candidates):
    return min(candidates, key=lambda e: sp.count_ops(e, visual=False))


class GroupBy(LayoutBlock):
    """Logical index space ``group_dims`` over a chain of physical orderings
    (reference: lego/lego.py:365-487)."""

    def __init__(self, group_dims, objects, user_constraints=[]):
        self._dims = tuple(d for level in group_dims for d in level)
        self.objects = objects
        self.d = len(group_dims[0])
        self.user_constraints = user_constraints
        self.constraints = {}

    def dims(self):
        return self._dims

    # raw maps (ints, arrays or expressions; nothing is simplified) ------------
    def apply(self, *idx):
        if len(idx) != len(self._dims):
            raise ValueError(
                f"Input index dimension mismatch. Expected {len(self._dims)}, got {len(idx)}")
        flat = flatten_index(idx, self._dims)
        for obj in reversed(self.objects):
            flat = obj.apply(unflatten_index(flat, obj.dims()))
        return flat

    def inv_raw(self, flat_idx):
        """Logical index of physical offset ``flat_idx`` without simplification."""
        flat = flat_idx
        for obj in self.objects:
            if not obj.dims():
                continue
            flat = flatten_index(obj.inv(flat), obj.dims())
        return unflatten_index(flat, self._dims)

    # simplified symbolic maps ----------------------------------------------------
    def _get_input_constraints(self):
        """Every size symbol is a positive integer (reference: lego/lego.py:439-441)."""
        found = set()
        for dims in [self._dims] + [o.dims() for o in self.objects]:
            for e in dims:
                if isinstance(e, sp.Expr):
                    found |= e.free_symbols
        return [sp.Gt(s, 0, evaluate=False) for s in sorted(found, key=str)]

    def _simplified(self, expr, facts, facts_for_expanded):
        return _fewer_ops(simplify_ops(expr, self.constraints, facts),
                          simplify_ops(sp.expand(expr), self.constraints, facts_for_expanded))

    def inv(self, flat_idx):
        facts = self._get_input_constraints() + list(self.user_constraints)
        logical = sp.sympify(self.inv_raw(flat_idx))
        self.constraints = {flat_idx: (0, product(self._dims))}
        return [self._simplified(component, facts, facts) for component in logical]

    def __getitem__(self, key):
        """Simplified flat offset of a logical index.

        Key grammar (reference: lego/lego.py:443-481): a slice is a whole axis
        (``TritonRange`` of ``tl.arange``); a string names an integer symbol; a sympy
        expression or an int is used as is.  Everything is assumed in range of its
        logical dimension.
        """
        if not isinstance(key, tuple):
            key = (key,)
        facts = self._get_input_constraints() + list(self.user_constraints)
        self.constraints = {}
        restore = {}
        index = []
        lane_rank = len(self.objects[0].dims())
        for position, item in enumerate(key):
            extent = self._dims[position]
            if isinstance(item, slice):
                lo = 0 if item.start is None else item.start
                hi = extent if item.stop is None else item.stop
                item = TritonRange(get_arange(lo, hi), position % lane_rank, lane_rank)
                bounds = (lo, hi)
            elif isinstance(item, str):
                s = sp.Symbol(item, integer=True)
                self.constraints[s] = (0, extent)
                index.append(s)
                continue
            elif isinstance(item, sp.Expr):
                bounds = (0, extent)
            else:
                index.append(item)  # a plain number addresses itself
                continue
            dummy = sp.Symbol(f"_tr{len(restore)}", integer=True)
            restore[dummy] = item
            self.constraints[dummy] = bounds
            index.append(dummy)
        flat = sp.sympify(self.apply(*index))
        # the expanded candidate is simplified from ranges alone, as in the reference
        return self._simplified(flat, facts, None).xreplace(restore)


# ---------------------------------------------------------------------------
# stock GenP bijections
# ---------------------------------------------------------------------------

def antidiag(n, args):
    """Anti-diagonal enumeration of an ``n x n`` square (reference: lego/lego.py:490-506)."""
    i, j = args
    d = i + j + 1
    upper = d * (d - 1) // 2 + i
    lower = (n * n - n) + i - ((2 * n - d) * (2 * n - d - 1) // 2)
    return Piecewise((upper, d <= n), (lower, True))


def antidiag_inv(n, x0):
    """Numeric inverse of ``antidiag`` (reference: lego/lego.py:509-530)."""
    first = n * (n + 1) // 2
    if x0 < first:
        k = math.floor((math.sqrt(8 * x0 + 1) - 1) / 2) + 1
        i = x0 - (k * (k - 1) // 2)
        return (i, (k - 1) - i)
    m = x0 - first
    d = math.floor((2 * n - 1 - math.sqrt((2 * n - 1) ** 2 - 8 * m)) / 2) + 1
    before = (d - 1) * n - ((d - 1) * d // 2)
    i = d + (m - before)
    return (i, (n + d - 1) - i)


def new_antidiag(n1, n2, args):
    i, j = args
    return (n1 - 1 - i) * n2 + n2 - 1 - j


class XorSwizzle:
    """``(r, c) -> r*cols + (c ^ ((r // every) % span) * unit)``: the row-dependent column
    rotation that spreads a tile's columns over LDS banks.

    ``unit`` consecutive columns move together (a 16-byte vector stays contiguous), a
    new rotation starts ``every`` rows, and ``span`` rotations exist.  ``span*unit`` must
    be a power of two that divides ``cols``, which makes the map an involution on the
    column digit and hence a bijection of the tile.  It is its own inverse on columns.
    """

    def __init__(self, rows, cols, unit=1, every=1, span=None):
        span = cols // unit if span is None else span
        for name, v in (("unit", unit), ("span", span)):
            if v & (v - 1):
                raise ValueError(f"{name} must be a power of two")
        if cols % (span * unit):
            raise ValueError("span*unit must divide cols")
        self.rows, self.cols, self.unit, self.every, self.span = rows, cols, unit, every, span

    def _key(self, r):
        return ((r // self.every) % self.span) * self.unit

    def apply(self, idx):
        r, c = idx
        return r * self.cols + _xor(c, self._key(r))

    def inv(self, flat):
        r, c = flat // self.cols, flat % self.cols
        return (r, _xor(c, self._key(r)))


def _xor(a, b):
    if isinstance(a, sp.Expr) or isinstance(b, sp.Expr):
        return BitXor(sp.sympify(a), sp.sympify(b))
    return a ^ b


def xor_swizzle(rows, cols, unit=1, every=1, span=None):
    """``GenP`` block holding an ``XorSwizzle`` of a ``rows x cols`` tile."""
    sw = XorSwizzle(rows, cols, unit, every, span)
    return GenP((rows, cols), sw.apply, sw.inv)
