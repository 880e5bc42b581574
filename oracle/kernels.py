"""TEST INFRASTRUCTURE -- CPU oracle for the five lego_hip kernels.  Not part of the product.

The reference's CPU path is "index expressions printed by ``lego_python`` and evaluated
over index vectors, plus PyTorch CPU operators".  Each function restates one kernel that
way and names what it follows:

``transpose``      benchmarks/mlir/transpose_smem.py:28-80 -- ``B[wby,wbx,i,j,..] = A[rby,rbx,j,i,..]``
                   over all logical indices, i.e. a gather/scatter through two layouts;
                   the reference's own check is ``gold[j*nx+i] = in[i*nx+j]``
                   (mlir_generated/transpose/transpose.cu:199-206).
``softmax``        triton_generated/softmax/softmax.py:33-58, checked there against
                   ``torch.softmax(x, axis=1)`` (:237-241).
``layernorm_fwd``  triton_generated/layernorm/layernorm.py:57-101 (mean, biased variance,
                   ``rstd = 1/sqrt(var+eps)``, ``y = (x-mean)*rstd*w + b``), checked there
                   against ``torch.nn.functional.layer_norm`` (:446).
``gemm``           triton_generated/matmul/matmul_NTA_NTB.py:97-122, checked against
                   ``torch.matmul`` (:252).
``grouped_gemm``   triton_generated/grouped_gemm/grouped_gemm.py:38-116, per problem
                   ``torch.matmul`` (:316-350).

Floating point oracles accumulate in fp32 and round once to fp16, which is what the
tolerances of the parity tests are stated against.
"""
from __future__ import annotations

import numpy as np
import torch

from . import lego_index as li


def transpose_layouts(rows, cols, tile_r, tile_c):
    """Source (row-major) and destination (column-major) tiled layouts of a
    ``rows x cols`` matrix, logical index ``(tile_i, tile_j, i, j)``."""
    levels = ([rows // tile_r, cols // tile_c], [tile_r, tile_c])
    return (li.tile_by(li.Order(li.row(rows, cols)), *levels),
            li.tile_by(li.Order(li.col(rows, cols)), *levels))


def transpose(x: torch.Tensor, tile_r: int, tile_c: int) -> torch.Tensor:
    """Move every element from its offset in the row-major layout to the offset of the
    same logical index in the column-major layout.  The result, read as a row-major
    ``cols x rows`` matrix, is the transpose."""
    rows, cols = x.shape
    src, dst = transpose_layouts(rows, cols, tile_r, tile_c)
    out = torch.empty(rows * cols, dtype=x.dtype)
    src_off = torch.from_numpy(np.array(src.offsets()).reshape(-1))
    dst_off = torch.from_numpy(np.array(dst.offsets()).reshape(-1))
    out[dst_off] = x.reshape(-1)[src_off]
    return out.view(cols, rows)


def softmax(x: torch.Tensor) -> torch.Tensor:
    return torch.softmax(x.float(), dim=-1).to(x.dtype)


def layernorm_fwd(x, weight, bias, eps=1e-5):
    """Returns ``(y, mean, rstd)`` with fp32 statistics."""
    xf = x.float()
    mean = xf.mean(dim=-1)
    var = xf.var(dim=-1, unbiased=False)
    rstd = torch.rsqrt(var + eps)
    y = torch.nn.functional.layer_norm(xf, (x.shape[-1],), weight.float(), bias.float(), eps)
    return y.to(x.dtype), mean, rstd


def layernorm_fwd_unrounded(x, weight, bias, eps=1e-5):
    """``y`` of :func:`layernorm_fwd` in fp32, before it is rounded to the tensors' type (what the
    reference's kernel holds in registers before its store, layernorm.py:94-101)."""
    return torch.nn.functional.layer_norm(x.float(), (x.shape[-1],), weight.float(), bias.float(), eps)


def half_spacing(y32: torch.Tensor, dtype) -> torch.Tensor:
    """Half the distance between neighbouring ``dtype`` values around each fp32 value: what a
    correctly rounded ``dtype`` result may differ from the fp32 value by."""
    bits, emin = {torch.float16: (10, -14), torch.bfloat16: (7, -126)}[dtype]
    expo = torch.floor(torch.log2(y32.abs().clamp(min=2.0 ** emin)))
    return torch.exp2(expo - bits - 1)


def gemm(a: torch.Tensor, b: torch.Tensor) -> torch.Tensor:
    return (a.float() @ b.float()).to(a.dtype)


def grouped_gemm(group_a, group_b):
    return [gemm(a, b) for a, b in zip(group_a, group_b)]


def grouped_pid(pid, num_pid_m, num_pid_n, group_m):
    """Textbook grouped launch order (triton_generated/matmul/matmul_NTA_NTB.py:176-181)."""
    width = group_m * num_pid_n
    group_id = pid // width
    first_m = group_id * group_m
    size_m = np.minimum(num_pid_m - first_m, group_m)
    return first_m + (pid % width) % size_m, (pid % width) // size_m


def needleman_wunsch(reference, penalty):
    """Rodinia's Needleman-Wunsch recurrence as the reference's kernels state it per cell
    (benchmarks/cuda/nw/needle_kernel_temp.cu:70-258: ``maximum(nw + ref, w - penalty, n - penalty)`` over
    the anti-diagonals of a tile; host loop and borders benchmarks/cuda/nw/needle.cu:165-260): borders
    ``-i*penalty``, then
    ``m[i][j] = max(m[i-1][j-1] + ref[i][j], m[i][j-1] - penalty, m[i-1][j] - penalty)``,
    evaluated one anti-diagonal at a time with numpy.  ``reference`` is ``(n+1) x (n+1)`` int32."""
    ref = np.asarray(reference, dtype=np.int64)
    n1 = ref.shape[0]
    m = np.zeros((n1, n1), dtype=np.int64)
    m[:, 0] = -np.arange(n1) * penalty
    m[0, :] = -np.arange(n1) * penalty
    for d in range(2, 2 * n1 - 1):                       # cells with i + j == d, i, j >= 1
        i = np.arange(max(1, d - (n1 - 1)), min(d - 1, n1 - 1) + 1)
        j = d - i
        m[i, j] = np.maximum(np.maximum(m[i - 1, j - 1] + ref[i, j], m[i, j - 1] - penalty), m[i - 1, j] - penalty)
    return m.astype(np.int32)


def bricks_order(n, b=8):
    """Offsets of the ``n^3`` points in bricks storage (benchmarks/cuda/bricks_f3d.py:11-12):
    ``OrderBy(Row(n/b, n/b, n/b), Row(b, b, b)).TileBy([n/b]*3, [b]*3)`` evaluated for every point,
    as an int64 array of shape ``(n, n, n)`` indexed by global coordinates."""
    nb = n // b
    lay = li.tile_by(li.Order(li.row(nb, nb, nb), li.row(b, b, b)), [nb, nb, nb], [b, b, b])
    off = lay.offsets()                                # indexed [bx, by, bz, i, j, k]
    return np.ascontiguousarray(off.transpose(0, 3, 1, 4, 2, 5)).reshape(n, n, n)


def stencil_f3d(x, c, radius):
    """The dense stencil of benchmarks/cuda/bricks/main_tmp.cu:24-66 on a row-major float32 array (a cube,
    or any box: a slab of a cube gives the cube's values on its inner planes), in float64: the centre
    is weighted once on its own and once more inside the window sum, boundary points are zero."""
    x = np.asarray(x, dtype=np.float64)
    c = np.asarray(c, dtype=np.float64)
    (n0, n1, n2), r = x.shape, radius
    out = np.zeros_like(x)
    core = (slice(r, n0 - r), slice(r, n1 - r), slice(r, n2 - r))
    acc = x[core] * c[r, r, r]
    for di in range(-r, r + 1):
        for dj in range(-r, r + 1):
            for dk in range(-r, r + 1):
                acc = acc + x[r + di:n0 - r + di, r + dj:n1 - r + dj, r + dk:n2 - r + dk] * c[di + r, dj + r, dk + r]
    out[core] = acc
    return out


def stencil_laplacian(x, c, radius):
    """The star stencil of benchmarks/cuda/bricks-laplace/main_tmp.cu:24-57, in float64 (cube or box)."""
    x = np.asarray(x, dtype=np.float64)
    c = np.asarray(c, dtype=np.float64)
    (n0, n1, n2), r = x.shape, radius
    out = np.zeros_like(x)
    core = (slice(r, n0 - r), slice(r, n1 - r), slice(r, n2 - r))
    i, j, k = core
    sh = lambda s_, a: slice(s_.start + a, s_.stop + a)      # noqa: E731
    acc = x[core] * c[0]
    for a in range(1, r + 1):
        acc = acc + c[a] * (x[sh(i, a), j, k] + x[sh(i, -a), j, k] + x[i, sh(j, a), k] + x[i, sh(j, -a), k]
                            + x[i, j, sh(k, a)] + x[i, j, sh(k, -a)])
    out[core] = acc
    return out


def lud(a):
    """LU decomposition without pivoting (Doolittle, unit lower triangle), what Rodinia's
    ``lud_base`` computes (the reference's CPU check, benchmarks/cuda/lud/lud.cu with common.c), in
    float64: returns one matrix with L below the diagonal and U on and above it."""
    m = np.array(a, dtype=np.float64)
    n = m.shape[0]
    for k in range(n - 1):
        m[k + 1:, k] /= m[k, k]
        m[k + 1:, k + 1:] -= np.outer(m[k + 1:, k], m[k, k + 1:])
    return m
