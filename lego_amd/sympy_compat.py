"""Guards against a sympy defect that corrupts index expressions.

sympy 1.14's ``Mod.eval`` rebuilds a product ``p`` from a list that already contains the
``Mod`` factors of ``p`` and then appends those factors again, so
``Mod(8*Mod(y, 2048), 256)`` evaluates to ``8*Mod(Mod(y, 2048)**2, 32)`` -- a different
function of ``y``.  Layout inverses produce exactly this shape (a digit times a stride,
reduced by another stride).  ``install()`` wraps ``Mod.eval`` so that, for an integer modulus
and a product with ``Mod`` factors, the evaluation runs on a copy of ``p`` whose ``Mod``
factors are opaque integer symbols; the factors are put back afterwards.  On sympy versions
without the defect the wrapper changes nothing.
"""
from __future__ import annotations

import sympy as sp
from sympy.core.mod import Mod

_installed = False


def _restore(expr, show):
    """Put the hidden ``Mod`` factors back, bottom up; a ``Mod`` node that would again be a
    product with ``Mod`` factors under an integer modulus is rebuilt unevaluated (it is
    already as simple as the evaluation above could make it)."""
    if expr in show:
        return show[expr]
    if not expr.args:
        return expr
    args = [_restore(a, show) for a in expr.args]
    if isinstance(expr, Mod):
        a, b = args
        if isinstance(a, sp.Mul) and b.is_Integer and any(isinstance(f, Mod) for f in a.args):
            return Mod(a, b, evaluate=False)
    return expr.func(*args)


def install():
    global _installed
    if _installed:
        return
    original = Mod.eval.__func__

    def guarded(cls, p, q):
        if isinstance(p, sp.Mul) and getattr(q, "is_Integer", False) and any(isinstance(a, Mod) for a in p.args):
            hide = {a: sp.Dummy("m", integer=True, nonnegative=bool(a.is_nonnegative))
                    for a in p.args if isinstance(a, Mod)}
            show = {d: a for a, d in hide.items()}
            res = original(cls, p.xreplace(hide), q)
            if res is None:
                return None
            return _restore(res, show)
        return original(cls, p, q)

    Mod.eval = classmethod(guarded)
    _installed = True
