"""C expression printer for LEGO index expressions (reference: lego/lego_c.py:5-38).

Integer semantics throughout: ``floor(a/b)`` is ``/`` on non-negative ints, ``x**2`` is
``x*x``.  Unlike the reference, which inherits ``fmin``/``fmax`` from the C99 printer,
``Min``/``Max`` are printed as integer ternaries, because index expressions are integers.
"""
from sympy.printing.c import C99CodePrinter
from sympy.printing.precedence import precedence

from .lego import *  # noqa: F401,F403


class NegativeProductMixin:
    """Prints ``-c*x`` as ``-`` followed by the product ``c*x``.

    sympy's code printers compute the parenthesisation level of a product before they strip
    its minus sign; a negative product therefore prints its factors at the level of a sum and
    ``x - 4*Mod(r, 2)`` comes out as ``x - 4*r % 2``, which C and Python read as
    ``x - (4*r) % 2``.  Printing the positive product on its own keeps the parentheses."""

    def _print_Mul(self, expr):
        coeff, _ = expr.as_coeff_Mul()
        if coeff.is_negative:
            positive = -expr
            text = self._print(positive)
            return "-(" + text + ")" if isinstance(positive, sp.Mod) else "-" + text
        return super()._print_Mul(expr)


class LEGOCCodePrinter(NegativeProductMixin, C99CodePrinter):
    def __init__(self, settings=None, **kwargs):
        merged = dict(settings or {})
        merged.update(kwargs)
        super().__init__(merged)

    def _print_floor(self, expr):
        num, den = expr.args[0].as_numer_denom()
        return f"(({self._print(num)})/({self._print(den)}))"

    def _print_Pow(self, expr):
        # small integer powers as products, as the reference prints them (`i*i`,
        # benchmarks/cuda/nw/needle_kernel.cu:10)
        if self._is_product_power(expr):
            base = self.parenthesize(expr.base, precedence(expr))
            return "*".join([base] * int(expr.exp))
        return super()._print_Pow(expr)

    @staticmethod
    def _is_product_power(expr):
        return expr.is_Pow and expr.exp.is_Integer and 2 <= int(expr.exp) <= 4

    def _print_Mod(self, expr):
        # An operand that is printed as a product must be parenthesised even though sympy ranks
        # a Pow above `%`: `Mod(w, n**2)` is `w % (n*n)`, not `w % n*n`.
        prec = precedence(expr)
        parts = []
        for arg in expr.args:
            text = self.parenthesize(arg, prec)
            if self._is_product_power(arg):
                text = f"({text})"
            parts.append(text)
        return " % ".join(parts)

    def _fold_minmax(self, args, op):
        out = self._print(args[0])
        for a in args[1:]:
            b = self._print(a)
            out = f"(({out}) {op} ({b}) ? ({out}) : ({b}))"
        return out

    def _print_Min(self, expr):
        return self._fold_minmax(expr.args, "<")

    def _print_Max(self, expr):
        return self._fold_minmax(expr.args, ">")

    def _print_BitXor(self, expr):
        a, b = expr.args
        return f"(({self._print(a)}) ^ ({self._print(b)}))"
