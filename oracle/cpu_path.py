"""TEST INFRASTRUCTURE -- the reference's CPU path, timed by bench.py as the CPU baseline and
checked by the tests.  Not part of the product.

LEGO's CPU path is "the index text its Python/Triton printer emits, evaluated over index vectors,
plus PyTorch CPU operators" (lego/lego_python.py:5-37: ``floor`` prints as ``//``, a
``TritonRange`` as a broadcast slice of ``tl.arange``; the generated kernels paste that text next
to ``tl.load``/``tl.store``, e.g. triton_generated/softmax/softmax.py:39,54).  On the CPU
``torch.arange`` stands in for ``tl.arange`` and a gather/scatter for the load/store pair.
"""
from __future__ import annotations

import types

import torch


def evaluate(text: str, **names) -> torch.Tensor:
    """Evaluate printed Python/Triton index text with int64 torch vectors for ``tl.arange``."""
    tl = types.SimpleNamespace(arange=lambda lo, hi: torch.arange(int(lo), int(hi), dtype=torch.int64))
    return eval(text, {"tl": tl, "min": min, "max": max, "__builtins__": {}}, names)


def transpose_printed(x: torch.Tensor, src_text: str, dst_text: str, tile_r: int, tile_c: int,
                      total_rows: int | None = None) -> torch.Tensor:
    """``out.view(-1)[dst] = x.view(-1)[src]`` with ``src``/``dst`` the printed offsets of every
    logical index ``(bi, bj, i, j)`` of a ``rows x cols`` panel: the first ``rows`` rows of a
    ``total_rows x cols`` row-major matrix (the whole matrix by default).  Returns the
    ``cols x rows`` panel of the transposed matrix's first ``rows`` columns, contiguous.

    The printed text names the matrix extents ``R`` and ``C`` and the numbers of tile rows and
    columns taken, ``nbi`` and ``nbj`` (benchmarks/mlir/transpose_smem.py:28-80 states the same copy
    per thread)."""
    rows, cols = x.shape
    total_rows = rows if total_rows is None else total_rows
    names = dict(R=total_rows, C=cols, nbi=rows // tile_r, nbj=cols // tile_c)
    src = evaluate(src_text, **names).reshape(-1)
    dst = evaluate(dst_text, **names).reshape(-1)
    # the destination is the whole transposed matrix (cols x total_rows); the panel's elements
    # land in its first `rows` columns
    col = dst % total_rows
    row = dst // total_rows
    out = torch.empty(cols * rows, dtype=x.dtype)
    out[row * rows + col] = x.reshape(-1)[src]
    return out.view(cols, rows)
