"""Range-based simplification of integer ``floor``/``Mod`` index expressions.

LEGO layouts produce nests of ``floor(x/d)`` and ``Mod(x, d)`` whenever a flat
offset is unfolded into digits and folded back in another order.  The reference
removes them with sympy pattern rules whose side conditions are discharged by z3
(reference: lego/z3_simplifier.py:266-386, entry point ``simplify_ops``).  This
module keeps the entry point and its contract -- the result has the same value
as the input for every assignment that satisfies the ranges -- but decides the
side conditions with a self-contained prover:

* every ranged symbol gets a closed symbolic interval; every other symbol is a
  size parameter (a positive integer);
* an expression's interval is obtained by monotone substitution, so the proof
  obligation ``0 <= r < d`` becomes the sign of a parameter-only expression;
* that sign is decided by clearing positive denominators, shifting every
  parameter ``p >= 1`` to ``1 + p'`` and checking that all coefficients of the
  expanded polynomial are non-negative.

The procedure is sound and incomplete: an obligation that it cannot discharge
leaves the ``floor``/``Mod`` in place, which changes the size of the generated
code and never its value.
"""
from __future__ import annotations

import sympy as sp
from sympy import Add, Integer, Mod, Mul, Pow, Rational, floor

from . import sympy_compat

sympy_compat.install()

__all__ = ["simplify_ops", "RangeProver", "BitXor"]


class BitXor(sp.Function):
    """Integer bitwise exclusive-or, ``BitXor(a, b) == a ^ b``.

    ``sympy.Xor`` is boolean; bank-conflict-free LDS swizzles need the integer
    operation inside a ``GenP`` block, so it is modelled as an opaque integer
    function that folds on integer literals and is printed as ``^``.
    """

    nargs = 2
    is_integer = True
    is_nonnegative = True

    @classmethod
    def eval(cls, a, b):
        if a.is_Integer and b.is_Integer:
            return Integer(int(a) ^ int(b))
        if b.is_zero:
            return a
        if a.is_zero:
            return b
        return None


def _pow2_cover(hi: int) -> int:
    """Smallest ``2**k - 1`` that is ``>= hi``."""
    return (1 << max(int(hi), 0).bit_length()) - 1


class RangeProver:
    """Decides ``e >= 0``, ``e < d``, ``d > 0`` and ``d != 0`` from symbol ranges.

    ``ranges`` maps a symbol (or, as the reference allows at lego/lego.py:421, an
    arbitrary index expression) to a half-open interval ``(lo, hi)``.  ``facts``
    are relationals as built by ``le_constraint`` / ``divisibility_constraint`` /
    ``sp.Gt(x, 0)``: a strict upper bound on a symbol tightens its interval, a
    positivity fact marks a parameter, a divisibility fact ``a % b == 0`` lets
    ``a/b`` count as an integer.
    """

    def __init__(self, ranges, facts=()):
        self.lo = {}
        self.hi = {}  # inclusive
        self.expr_ranges = []
        self.positive = set()
        self.divides = set()  # (a, b): b divides a
        for key, (lo, hi) in ranges.items():
            key = sp.sympify(key)
            lo, hi = sp.sympify(lo), sp.sympify(hi)
            if key.is_Symbol:
                self.lo[key] = lo
                self.hi[key] = hi - 1
            elif not key.is_number:
                self.expr_ranges.append((key, lo, hi - 1))
        for f in facts or ():
            self._absorb(f)
        self._memo = {}
        self._bmemo = {}

    # -- facts ---------------------------------------------------------------
    def _absorb(self, f):
        if isinstance(f, sp.StrictGreaterThan):
            f = sp.StrictLessThan(f.rhs, f.lhs, evaluate=False)
        elif isinstance(f, sp.GreaterThan):
            f = sp.LessThan(f.rhs, f.lhs, evaluate=False)
        if isinstance(f, sp.StrictLessThan):
            a, b = f.lhs, f.rhs
            if a.is_Symbol and not b.has(a):
                self._tighten_hi(a, b - 1)
            if b.is_Symbol and not a.has(b):
                self._tighten_lo(b, a + 1)
            if a == 0 and b.is_Symbol:
                self.positive.add(b)
        elif isinstance(f, sp.LessThan):
            a, b = f.lhs, f.rhs
            if a.is_Symbol and not b.has(a):
                self._tighten_hi(a, b)
            if b.is_Symbol and not a.has(b):
                self._tighten_lo(b, a)
        elif isinstance(f, sp.Equality):
            a, b = f.lhs, f.rhs
            if isinstance(a, Mod) and b == 0:
                self.divides.add((a.args[0], a.args[1]))
            elif a.is_Symbol and not b.has(a):
                self._tighten_lo(a, b)
                self._tighten_hi(a, b)

    def _tighten_hi(self, s, v):
        # a range given for the symbol itself wins over a user fact
        self.hi.setdefault(s, v)
        if s not in self.lo and (s.is_nonnegative or s.is_positive):
            self.lo[s] = Integer(1) if s.is_positive else Integer(0)

    def _tighten_lo(self, s, v):
        if s in self.hi or s in self.lo:
            self.lo.setdefault(s, v)
        # a lower bound alone does not turn a parameter into a ranged index

    # -- parameters ------------------------------------------------------------
    def _is_param_positive(self, a):
        if a in self.positive or a.is_positive:
            return True
        if isinstance(a, (sp.Min, sp.Max)):
            return all(self.sign_positive(x) for x in a.args)
        return False

    # -- intervals -------------------------------------------------------------
    def bounds(self, e):
        """Inclusive ``(lo, hi)`` of ``e`` as parameter-only expressions, or ``None``
        for a side that is not known."""
        e = sp.sympify(e)
        hit = self._bmemo.get(e)
        if hit is None:
            hit = self._bounds(e)
            self._bmemo[e] = hit
        return hit

    def _is_ranged(self, e):
        if e.free_symbols & (set(self.hi) | set(self.lo)):
            return True
        return any(e.has(key) for key, _, _ in self.expr_ranges)

    def _bounds(self, e):
        if e.is_number:
            return (e, e)
        if not e.is_Symbol and not self._is_ranged(e):
            return (e, e)  # a parameter-only expression is its own exact bound
        if e.is_Symbol:
            if e in self.hi or e in self.lo:
                lo, hi = self.lo.get(e), self.hi.get(e)
                # a bound may itself mention ranged symbols (tid < T*T is fine,
                # j < i would not be parameter-only): resolve one level.
                if lo is not None and lo.free_symbols & (set(self.hi) | set(self.lo)):
                    lo = self.bounds(lo)[0] if e not in lo.free_symbols else None
                if hi is not None and hi.free_symbols & (set(self.hi) | set(self.lo)):
                    hi = self.bounds(hi)[1] if e not in hi.free_symbols else None
                return (lo, hi)
            return (e, e)
        for key, lo, hi in self.expr_ranges:
            if e == key:
                return (lo, hi)
        if isinstance(e, Add):
            los, his = [], []
            for a in e.args:
                lo, hi = self.bounds(a)
                los.append(lo)
                his.append(hi)
            return (None if None in los else Add(*los), None if None in his else Add(*his))
        if isinstance(e, Mul):
            coeff, rest = e.as_coeff_Mul()
            if coeff.is_negative:
                lo, hi = self.bounds(-e)
                return (None if hi is None else -hi, None if lo is None else -lo)
            lo_acc, hi_acc = Integer(1), Integer(1)
            for a in e.args:
                lo, hi = self.bounds(a)
                if lo is None or not self.sign_nonneg(lo):
                    return (None, None)
                lo_acc = lo_acc * lo
                hi_acc = None if (hi is None or hi_acc is None) else hi_acc * hi
            return (lo_acc, hi_acc)
        if isinstance(e, Pow):
            base, ex = e.args
            if ex.is_Integer:
                lo, hi = self.bounds(base)
                if lo is not None and hi is not None and self.sign_positive(lo):
                    n = int(ex)
                    if n > 0:
                        return (lo ** n, hi ** n)
                    return (hi ** n, lo ** n)
            return (None, None)
        if isinstance(e, floor):
            lo, hi = self.bounds(e.args[0])
            if lo is not None:
                lo = floor(lo) if lo.is_number else (Integer(0) if self.sign_nonneg(lo) else None)
            if hi is not None and hi.is_number:
                hi = floor(hi)
            elif hi is not None:
                # floor((q*d + r)/d) = q + floor(r/d): with r = -1 and d >= 1 that is q - 1,
                # the usual "largest digit" bound of a flat index divided by a stride
                num, den = sp.together(hi).as_numer_denom()
                if not den.is_number and self.sign_positive(den):
                    quot, rest = [], []
                    for term in Add.make_args(sp.expand(num)):
                        q = sp.cancel(term / den)
                        (quot if q.is_integer else rest).append(q if q.is_integer else term)
                    r = Add(*rest)
                    if quot and r.is_number and r < 0 and self.sign_nonneg(den + r):
                        hi = Add(*quot) - 1
            return (lo, hi)
        if isinstance(e, Mod):
            x, d = e.args
            dlo, dhi = self.bounds(d)
            if dlo is not None and dhi is not None and self.sign_positive(dlo):
                xlo, xhi = self.bounds(x)
                if xlo is not None and xhi is not None and self.sign_nonneg(xlo) \
                        and self.sign_positive(dlo - xhi):
                    return (xlo, xhi)
                return (Integer(0), dhi - 1)
            return (None, None)
        if isinstance(e, (sp.Min, sp.Max)):
            parts = [self.bounds(a) for a in e.args]
            los = [p[0] for p in parts]
            his = [p[1] for p in parts]
            return (None if None in los else e.func(*los), None if None in his else e.func(*his))
        if isinstance(e, BitXor):
            parts = [self.bounds(a) for a in e.args]
            if all(p[0] is not None and p[1] is not None and p[1].is_number
                   and self.sign_nonneg(p[0]) for p in parts):
                return (Integer(0), Integer(_pow2_cover(max(int(p[1]) for p in parts))))
            return (None, None)
        if isinstance(e, sp.Piecewise):
            parts = [self.bounds(v) for v, _ in e.args]
            if all(p[0] is not None and p[1] is not None and p[0].is_number and p[1].is_number
                   for p in parts):
                return (min(p[0] for p in parts), max(p[1] for p in parts))
            return (None, None)
        return (None, None)

    # -- signs of parameter-only expressions --------------------------------------
    def _sign(self, d, strict):
        d = sp.sympify(d)
        if d.is_number:
            return bool(d > 0) if strict else bool(d >= 0)
        key = (d, strict)
        hit = self._memo.get(key)
        if hit is not None:
            return hit
        res = self._sign_uncached(d, strict)
        self._memo[key] = res
        return res

    def _sign_uncached(self, d, strict):
        if strict and d.is_positive:
            return True
        if not strict and d.is_nonnegative:
            return True
        if isinstance(d, (sp.Min,)):
            return all(self._sign(a, strict) for a in d.args)
        if isinstance(d, (sp.Max,)):
            return any(self._sign(a, strict) for a in d.args)
        num, den = sp.together(d).as_numer_denom()
        if not den.is_number:
            for f in Mul.make_args(den):
                base = f.args[0] if isinstance(f, Pow) else f
                if base.is_number:
                    if base < 0:
                        return False
                    continue
                if not (self._is_param_positive(base) or self._poly_sign(sp.expand(base), True)):
                    return False
        elif den < 0:
            num = -num
        return self._poly_sign(self._relax_negative_terms(sp.expand(num)), strict)

    @staticmethod
    def _relax_negative_terms(p):
        """Replace, in terms with a negative coefficient, products that have a simple
        upper bound by that bound; the result is ``<= p``, so its sign carries over.

        ``floor(a/b)*b <= a`` and ``Max(1, floor(a/b))*Min(a, b) <= a`` for positive
        integers: the second is the grouped launch order's "groups times group size
        never exceeds the tile count" (reference layout: benchmarks/triton/matmul_sympy.py:60-61).
        """
        out = []
        for t in Add.make_args(p):
            c, rest = t.as_coeff_Mul()
            if c < 0:
                factors = []
                for f in Mul.make_args(rest):
                    if isinstance(f, Pow) and f.exp.is_Integer and 1 < int(f.exp) <= 8:
                        factors += [f.base] * int(f.exp)
                    else:
                        factors.append(f)
                for f in list(factors):
                    inner = None
                    if isinstance(f, floor):
                        inner = f
                    elif isinstance(f, sp.Max) and len(f.args) == 2 and Integer(1) in f.args:
                        other = [x for x in f.args if x != 1][0]
                        if isinstance(other, floor):
                            inner = other
                    if inner is None:
                        continue
                    a, b = inner.args[0].as_numer_denom()
                    if not (a.is_positive and b.is_positive and a.is_integer and b.is_integer):
                        continue
                    partner = b if isinstance(f, floor) else sp.Min(a, b)
                    if partner in factors and f in factors:
                        factors.remove(f)
                        factors.remove(partner)
                        factors.append(a)
                rest = Mul(*factors)
            out.append(c * rest)
        return sp.expand(Add(*out))

    def _poly_sign(self, p, strict):
        """All-coefficients test after shifting parameters known to be >= 1."""
        if p.is_number:
            return bool(p > 0) if strict else bool(p >= 0)
        atoms = set()
        for t in Add.make_args(p):
            for f in Mul.make_args(t):
                base = f.args[0] if isinstance(f, Pow) else f
                if not base.is_number:
                    atoms.add(base)
        shift = {}
        for a in atoms:
            if a.is_Symbol and (a in self.hi or a in self.lo):
                return False  # a ranged symbol leaked into a parameter expression
            kind = self._atom_kind(a)
            if kind is None:
                return False
            if kind == "ge1":
                shift[a] = 1 + sp.Dummy(nonnegative=True)
        q = sp.expand(p.xreplace(shift)) if shift else p
        const = Integer(0)
        for t in Add.make_args(q):
            c, rest = t.as_coeff_Mul()
            if c < 0:
                return False
            if rest == 1:
                const = c
        return bool(const > 0) if strict else True

    def _atom_kind(self, a):
        """``"ge1"`` for a positive integer atom, ``"ge0"`` for a non-negative one."""
        if a.is_Symbol:
            if a in self.positive or a.is_positive:
                return "ge1" if a.is_integer else "ge0"
            return "ge0" if a.is_nonnegative else None
        if isinstance(a, floor):
            return "ge0" if self.sign_nonneg(a.args[0]) else None
        if isinstance(a, Mod):
            return "ge0" if self.sign_positive(a.args[1]) else None
        if isinstance(a, (sp.Min, sp.Max)):
            pick = all if isinstance(a, sp.Min) else any
            whole = all(x.is_integer for x in a.args)
            if whole and pick(self.sign_positive(x) for x in a.args):
                return "ge1"
            if pick(self.sign_nonneg(x) for x in a.args):
                return "ge0"
        return None

    def sign_positive(self, d):
        return self._sign(d, True)

    def sign_nonneg(self, d):
        return self._sign(d, False)

    # -- obligations -----------------------------------------------------------------
    def nonneg(self, e):
        lo, _ = self.bounds(e)
        return lo is not None and self.sign_nonneg(lo)

    def positive_(self, e):
        lo, _ = self.bounds(e)
        return lo is not None and self.sign_positive(lo)

    def less(self, e, d):
        _, hi = self.bounds(e)
        dlo, _ = self.bounds(d)
        return hi is not None and dlo is not None and self.sign_positive(dlo - hi)

    def in_range(self, r, d):
        """``0 <= r < d``."""
        return self.nonneg(r) and self.less(r, d)

    def can_prove(self, rel):
        """Decide a sympy relational; ``False`` means "not proven"."""
        if rel is True or rel == sp.true:
            return True
        if rel is False or rel == sp.false:
            return False
        if isinstance(rel, sp.StrictLessThan):
            return self.less(rel.lhs, rel.rhs)
        if isinstance(rel, sp.StrictGreaterThan):
            return self.less(rel.rhs, rel.lhs)
        if isinstance(rel, sp.GreaterThan):
            return self.nonneg(rel.lhs - rel.rhs)
        if isinstance(rel, sp.LessThan):
            return self.nonneg(rel.rhs - rel.lhs)
        if isinstance(rel, sp.Unequality):
            return self.positive_(rel.lhs - rel.rhs) or self.positive_(rel.rhs - rel.lhs)
        return False

    # -- integrality --------------------------------------------------------------------
    def integer_valued(self, q):
        """True when ``q`` takes integer values: an integer polynomial in integer atoms,
        possibly times ratios declared exact by a divisibility fact."""
        if q.is_integer:
            return True
        num, den = sp.cancel(q).as_numer_denom()
        if den == 1:
            return bool(num.is_integer)
        for a, b in self.divides:
            if sp.cancel(q * b / a).is_integer or sp.cancel(q / (a / b)).is_integer:
                return True
        return False


# ---------------------------------------------------------------------------------------
# rewriting
# ---------------------------------------------------------------------------------------

def _split_multiples(num, den, prover):
    """Write ``num`` as ``den*quot + rest`` term by term."""
    quot, rest = [], []
    for t in Add.make_args(sp.expand(num)):
        q = sp.cancel(t / den)
        if t != 0 and prover.integer_valued(q):
            quot.append(q)
        else:
            rest.append(t)
    return Add(*quot), Add(*rest)


def _num_den(x):
    num, den = sp.together(x).as_numer_denom()
    return sp.expand(num), sp.expand(den)


def _rewrite_floor(e, prover):
    x = e.args[0]
    num, den = _num_den(x)
    if den == 1:
        return num if num.is_integer else e
    if not prover.positive_(den):
        return e
    # floor(floor(a/b)/c) == floor(a/(b*c)) for positive integers b, c
    if isinstance(num, floor):
        inum, iden = _num_den(num.args[0])
        if prover.positive_(iden) and inum.is_integer is not False:
            return _rewrite_floor(floor(inum / (iden * den), evaluate=False), prover)
    quot, rest = _split_multiples(num, den, prover)
    if rest == 0:
        return quot
    if prover.in_range(rest, den):
        return quot
    # Mod(x, a*den) // den keeps only the high digit: nothing simpler to write
    # common numeric factor of numerator and denominator
    if den.is_Integer:
        g = sp.gcd(sp.gcd_list([t.as_coeff_Mul()[0] for t in Add.make_args(rest)]), den)
        if g != 1 and g == den:  # every coefficient is a multiple of den
            return quot + sp.expand(rest / den)
    return quot + floor(rest / den)


def _rewrite_mod(e, prover):
    x, d = e.args
    if not prover.positive_(d):
        return e
    _, rest = _split_multiples(x, d, prover)
    if rest == 0:
        return Integer(0)
    if prover.in_range(rest, d):
        return rest
    # Mod(Mod(y, k*d), d) == Mod(y, d)
    if isinstance(rest, Mod) and prover.integer_valued(sp.cancel(rest.args[1] / d)):
        return _rewrite_mod(Mod(rest.args[0], d, evaluate=False), prover)
    return Mod(rest, d)


def _recombine(e, prover):
    """``c*a*floor(x/a) + c*Mod(x, a) -> c*x`` among the terms of a sum."""
    args = list(Add.make_args(e))
    changed = True
    while changed:
        changed = False
        for i, t in enumerate(args):
            c, m = t.as_coeff_Mul()
            if not isinstance(m, Mod):
                continue
            x, a = m.args
            want = c * a * floor(x / a)
            for j, u in enumerate(args):
                if j != i and sp.expand(u - want) == 0 and prover.positive_(a):
                    args = [v for k, v in enumerate(args) if k not in (i, j)] + [c * x]
                    changed = True
                    break
            if changed:
                break
    return Add(*args)


def _walk(e, prover):
    if e.is_Atom:
        return e
    args = [_walk(a, prover) for a in e.args]
    if isinstance(e, floor):
        f = floor(args[0])  # sympy itself pulls integer terms out of the floor
        if isinstance(f, floor):
            return _rewrite_floor(f, prover)
        return f.replace(lambda n: isinstance(n, floor), lambda n: _rewrite_floor(n, prover))
    if isinstance(e, Mod):
        m = Mod(args[0], args[1])
        return _rewrite_mod(m, prover) if isinstance(m, Mod) else m
    if isinstance(e, sp.Piecewise):
        return e.func(*[(a.args[0], a.args[1]) for a in args]) if all(
            hasattr(a, "args") and len(a.args) == 2 for a in args) else e
    out = e.func(*args)
    if isinstance(out, Add):
        out = _recombine(out, prover)
    return out


def simplify_ops(expr, bounds, additional_bounds=None, var_types=None, timeout=None):
    """Value-preserving simplification of ``expr`` under ``bounds``.

    Same call surface as the reference's ``simplify_ops``
    (lego/z3_simplifier.py:367): ``bounds`` maps symbols to half-open ``(lo, hi)``
    intervals, ``additional_bounds`` is a list of relationals.  ``var_types`` and
    ``timeout`` are accepted for compatibility and unused (there is no solver).
    """
    prover = RangeProver(bounds, additional_bounds or ())
    cur = sp.sympify(expr)
    for _ in range(32):
        nxt = _walk(cur, prover)
        if nxt == cur:
            break
        cur = nxt
    return cur
