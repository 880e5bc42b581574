"""Python/Triton expression printer for LEGO index expressions.

The printed text, evaluated with ``numpy``/``torch`` standing in for ``tl``, is the CPU
index path of LEGO (reference: lego/lego_python.py:5-37): ``floor(a/b)`` becomes ``//``
and a ``TritonRange`` becomes a broadcast slice of its index vector.
"""
from sympy.printing.pycode import PythonCodePrinter

from .lego import *  # noqa: F401,F403
from .lego_c import NegativeProductMixin


class LEGOPythonCodePrinter(NegativeProductMixin, PythonCodePrinter):
    """``LEGOPythonCodePrinter(allow_unknown_functions=True, do_broadcast=True)``."""

    def __init__(self, settings=None, **kwargs):
        self.do_broadcast = kwargs.pop("do_broadcast", True)
        merged = dict(settings or {})
        merged.update(kwargs)
        super().__init__(merged)

    def _print_floor(self, expr):
        num, den = expr.args[0].as_numer_denom()
        return f"(({self._print(num)})//({self._print(den)}))"

    def _print_TritonRange(self, expr):
        vec, rank = expr.args[0], expr.args[2]
        if rank == 1 or not self.do_broadcast:
            return f"({vec})"
        return f"(({vec})[{expr.broadcast_suffix()}])"

    def _print_BitXor(self, expr):
        a, b = expr.args
        return f"(({self._print(a)}) ^ ({self._print(b)}))"
