"""Host entry points with the call signatures of the reference's generated host functions.

``softmax(x)``                       triton_generated/softmax/softmax.py:97-160
``lego_layer_norm(x, shape, w, b, eps)``  triton_generated/layernorm/layernorm.py:279-307, 407
``matmul(a, b, activation="")``      triton_generated/matmul/matmul_NTA_NTB.py:129-145
``lego_group_gemm_fn(group_A, group_B)``  triton_generated/grouped_gemm/grouped_gemm.py:120-162
``transpose(x)``                     the generated transpose programs have no callable
                                     (mlir_generated/transpose/transpose_smem_4096.mlir:2)

As in the reference, inputs are borrowed, outputs are allocated here with ``torch.empty``
and the kernel is enqueued on the current stream without synchronisation.  Tensors are
only carriers of device pointers: every call goes through the C ABI of liblego_hip.so.
"""
from __future__ import annotations

import ctypes

import torch

from . import runtime


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _stream():
    """The current stream's handle (an integer, or None for the null stream: what a ``c_void_p`` parameter takes);
    asked for on every call, since the caller may switch streams."""
    if _raw_stream is not None:      # without building a torch.cuda.Stream object
        return _raw_stream(torch.cuda.current_device()) or None
    return torch.cuda.current_stream().cuda_stream or None


def _ptr(t):
    """The tensor's address as an integer (None for an empty tensor's null pointer): a ``c_void_p`` parameter."""
    return t.data_ptr() or None


def _check(t, dtype, name, ndim=2):
    if not t.is_cuda:
        raise ValueError(f"{name} must live on the GPU")
    if t.dtype != dtype:
        raise ValueError(f"{name} must be {dtype}, got {t.dtype}")
    if t.dim() != ndim:
        raise ValueError(f"{name} must have {ndim} dimensions")
    if not t.is_contiguous():
        raise ValueError(f"{name} must be contiguous")


def transpose(x: torch.Tensor) -> torch.Tensor:
    """``x.T`` materialised: the ``rows x cols`` row-major input copied into the
    column-major layout of the same logical matrix."""
    if x.element_size() not in (2, 4):
        raise ValueError("transpose moves 2-byte and 4-byte elements (float16, bfloat16, float32, int32, ...)")
    _check(x, x.dtype, "x")
    rows, cols = x.shape
    out = torch.empty((cols, rows), device=x.device, dtype=x.dtype)
    # the kernels move bits: the entry point is chosen by element size
    entry = "lego_hip_transpose_f32" if x.element_size() == 4 else "lego_hip_transpose_f16"
    runtime.call(entry, _ptr(x), _ptr(out), rows, cols, _stream())
    return out


_ROW_TAG = {torch.float16: "f16", torch.bfloat16: "bf16", torch.float32: "f32"}


def softmax(x: torch.Tensor, waves_per_row: int | None = None) -> torch.Tensor:
    """Row softmax of a 2-D fp16, bf16 or fp32 tensor."""
    if x.dtype not in _ROW_TAG:
        raise ValueError("softmax supports float16, bfloat16 and float32")
    _check(x, x.dtype, "x")
    n_rows, n_cols = x.shape
    y = torch.empty_like(x)
    if waves_per_row is None:
        runtime.call(f"lego_hip_softmax_{_ROW_TAG[x.dtype]}", _ptr(x), _ptr(y), n_rows, n_cols, _stream())
    elif x.dtype != torch.float16:
        raise ValueError("waves_per_row is a tuning knob of the fp16 kernels")
    else:
        runtime.call("lego_hip_softmax_f16_wpr", _ptr(x), _ptr(y), n_rows, n_cols, waves_per_row, _stream())
    return y


def layer_norm_fwd(x, weight, bias, eps=1e-5, waves_per_row: int | None = None):
    """LayerNorm forward over the last dimension; returns ``(y, mean, rstd)``."""
    if x.dtype not in _ROW_TAG:
        raise ValueError("x must be float16, bfloat16 or float32")
    x_arg = x if x.dim() == 2 else x.reshape(-1, x.shape[-1])      # every torch call here costs a microsecond
    _check(x_arg, x.dtype, "x")
    M, N = x_arg.shape
    _check(weight, x.dtype, "weight", ndim=1)
    _check(bias, x.dtype, "bias", ndim=1)
    if weight.shape[0] != N or bias.shape[0] != N:
        raise ValueError("weight and bias must have the size of the normalised dimension")
    if N * x.element_size() > 65536:
        # the reference's limit and message (layernorm.py:293-294)
        raise RuntimeError("This layer norm doesn't support feature dim >= 64KB.")
    y = torch.empty_like(x_arg)
    mean = torch.empty((M,), dtype=torch.float32, device=x.device)
    rstd = torch.empty((M,), dtype=torch.float32, device=x.device)
    args = (_ptr(x_arg), _ptr(y), _ptr(weight), _ptr(bias), _ptr(mean), _ptr(rstd), M, N, float(eps))
    if waves_per_row is None:
        runtime.call(f"lego_hip_layernorm_fwd_{_ROW_TAG[x.dtype]}", *args, _stream())
    elif x.dtype != torch.float16:
        raise ValueError("waves_per_row is a tuning knob of the fp16 kernels")
    else:
        runtime.call("lego_hip_layernorm_fwd_f16_wpr", *args, waves_per_row, _stream())
    return (y if x.dim() == 2 else y.view(x.shape)), mean, rstd


_bwd_workspace = {}      # (element tag, M, N) -> bytes of fp32 partial sums


def layer_norm_bwd(dy, x, weight, mean, rstd):
    """LayerNorm backward; returns ``(dx, dw, db)``.  fp16, bf16 or fp32 tensors, rows of up to 32768 elements."""
    if x.dtype not in _ROW_TAG:
        raise ValueError("x must be float16, bfloat16 or float32")
    tag = _ROW_TAG[x.dtype]
    x_arg = x if x.dim() == 2 else x.reshape(-1, x.shape[-1])
    dy_arg = dy if dy.dim() == 2 and dy.is_contiguous() else dy.reshape(-1, dy.shape[-1]).contiguous()
    _check(x_arg, x.dtype, "x")
    _check(dy_arg, x.dtype, "dy")
    _check(weight, x.dtype, "weight", ndim=1)
    M, N = x_arg.shape
    if dy_arg.shape != x_arg.shape or weight.shape[0] != N:
        raise ValueError("dy must have the shape of x and weight the length of its rows")
    for name, stat in (("mean", mean), ("rstd", rstd)):
        _check(stat, torch.float32, name, ndim=1)       # the forward pass's fp32 statistics, one per row
        if stat.shape[0] != M or stat.device != x.device:
            raise ValueError(f"{name} must hold one float32 per row of x, on its device")
    need = _bwd_workspace.get((tag, M, N))
    if need is None:      # asked once per shape: the answer is a function of the shape alone
        size = ctypes.c_ulonglong(0)
        runtime.call("lego_hip_layernorm_bwd_workspace_bytes" if tag == "f16" else f"lego_hip_layernorm_bwd_{tag}_workspace_bytes",
                     M, N, ctypes.byref(size))
        if len(_bwd_workspace) >= 4096:
            _bwd_workspace.clear()
        need = _bwd_workspace[(tag, M, N)] = size.value
    # like the reference's wrapper, which allocates its partial buffers with torch (layernorm.py:381-383)
    workspace = torch.empty(need // 4, dtype=torch.float32, device=x.device)
    dx = torch.empty_like(x_arg)
    dw = torch.empty((N,), dtype=weight.dtype, device=x.device)
    db = torch.empty((N,), dtype=weight.dtype, device=x.device)
    runtime.call(f"lego_hip_layernorm_bwd_{tag}", _ptr(dy_arg), _ptr(x_arg), _ptr(weight), _ptr(mean), _ptr(rstd),
                 _ptr(dx), _ptr(dw), _ptr(db), _ptr(workspace), need, M, N, _stream())
    return (dx if x.dim() == 2 else dx.view(x.shape)), dw, db


class LEGOLayerNorm(torch.autograd.Function):
    """``lego_layer_norm = LEGOLayerNorm.apply`` with the reference's signature and gradients
    (triton_generated/layernorm/layernorm.py:323-405)."""

    @staticmethod
    def forward(ctx, x, normalized_shape, weight, bias, eps):
        if tuple(normalized_shape) != (x.shape[-1],):
            raise ValueError("normalized_shape must be the last dimension of x")
        y, mean, rstd = layer_norm_fwd(x, weight, bias, eps)
        ctx.save_for_backward(x, weight, bias, mean, rstd)
        ctx.eps = eps
        return y

    @staticmethod
    def backward(ctx, dy):
        x, w, b, m, v = ctx.saved_tensors
        dx, dw, db = layer_norm_bwd(dy, x, w, m, v)
        return dx, None, dw, db, None


lego_layer_norm = LEGOLayerNorm.apply


_GEMM_ENTRY = {torch.float16: "lego_hip_gemm_f16_ex", torch.bfloat16: "lego_hip_gemm_bf16_ex"}
_FP8_FORMAT = {torch.float8_e4m3fn: 0, torch.float8_e5m2: 1}


def _operand(t, name):
    """``(storage tensor, transposed?)`` of a 2-D fp16/bf16 operand that is contiguous either as
    given or as its transpose (the reference's TA/TB variants pass ``x.T`` views)."""
    if not t.is_cuda or (t.dtype not in _GEMM_ENTRY and t.dtype not in _FP8_FORMAT) or t.dim() != 2:
        raise ValueError(f"{name} must be a 2-D float16, bfloat16 or float8 GPU tensor")
    if t.is_contiguous():
        return t, 0
    if t.t().is_contiguous():
        return t.t(), 1
    raise ValueError(f"{name} must be contiguous or the transpose of a contiguous tensor")


_gemm_workspace = {}      # (M, N, K) -> bytes of workspace that lego_hip_gemm_ex_ws uses


def matmul(a: torch.Tensor, b: torch.Tensor, activation: str = "", out_dtype=torch.float16) -> torch.Tensor:
    """``act(a @ b)`` for fp16, bf16 or 8-bit floating-point operands of any shape, each row-major or
    column-major (a ``.T`` view), fp32 accumulation, row-major fp16 result: the reference's ``matmul``
    allocates a float16 result whatever its operands' type (matmul_sympy.py:129-145, its fp8 path
    :346-364).  ``out_dtype=torch.bfloat16`` with bfloat16 operands keeps their type instead."""
    if activation not in ("", "leaky_relu"):
        raise NotImplementedError(f"activation {activation!r} is not generated by this build")
    a_store, ta = _operand(a, "a")
    b_store, tb = _operand(b, "b")
    M, K = a.shape
    K2, N = b.shape
    if K != K2:
        raise ValueError("Incompatible dimensions")
    if a.dtype != b.dtype:
        raise ValueError("a and b must have the same dtype")
    if a.dtype in _FP8_FORMAT:
        c = torch.empty((M, N), device=a.device, dtype=torch.float16)
        runtime.call("lego_hip_gemm_fp8_ex", _ptr(a_store), _ptr(b_store), _ptr(c), M, N, K, ta, tb,
                     1 if activation else 0, _FP8_FORMAT[a.dtype], _stream())
        return c
    if out_dtype not in (torch.float16, a.dtype):
        raise ValueError("out_dtype must be float16 or the operands' type")
    entry = "lego_hip_gemm_bf16_f16_ex" if (a.dtype, out_dtype) == (torch.bfloat16, torch.float16) else _GEMM_ENTRY[a.dtype]
    if ta and M % 8 and M * K >= 65536:
        # a column-major A whose columns (M elements) are not whole 16-byte chunks is outside the tiled kernels whatever
        # the workspace: store it row-major first (one pass with the transpose kernels)
        a_store, ta = transpose(a_store), 0
    c = torch.empty((M, N), device=a.device, dtype=out_dtype)
    # products of few tiles (a skinny operand, a long K) are split along K when there is room for the partial sums;
    # shapes whose operand rows are not whole 16-byte chunks run on zero-padded copies in the workspace
    need = _gemm_workspace.get((M, N, K))
    if need is None:      # asked once per shape
        size = ctypes.c_ulonglong(0)
        runtime.call("lego_hip_gemm_workspace_bytes", M, N, K, ctypes.byref(size))
        if len(_gemm_workspace) >= 4096:
            _gemm_workspace.clear()
        need = _gemm_workspace[(M, N, K)] = size.value
    if need:
        workspace = torch.empty(need // 4, dtype=torch.float32, device=a.device)
        element = 0 if a.dtype == torch.float16 else 4 if out_dtype == torch.float16 else 1
        runtime.call("lego_hip_gemm_ex_ws", element, _ptr(a_store), _ptr(b_store), _ptr(c), M, N, K, ta, tb,
                     1 if activation else 0, _ptr(workspace), need, _stream())
        return c
    runtime.call(entry, _ptr(a_store), _ptr(b_store), _ptr(c), M, N, K, ta, tb, 1 if activation else 0, _stream())
    return c


def lego_group_gemm_fn(group_A, group_B):
    """One launch for a list of independent GEMMs; returns the list of results."""
    if len(group_A) != len(group_B):
        raise ValueError("group_A and group_B must have the same length")
    for a, b in zip(group_A, group_B):
        _check(a, torch.float16, "A")
        _check(b, torch.float16, "B")
        if a.shape[1] != b.shape[0]:
            raise ValueError("Incompatible dimensions")
    # Problems whose rows are not whole 16-byte chunks would take the whole call to one launch per problem with the
    # one-element kernel: those few go through ``matmul`` (zero-padded copies, a workspace from torch), the rest in
    # one launch.
    odd = [i for i, b in enumerate(group_B) if b.shape[0] % 8 or b.shape[1] % 8]
    if odd:
        rest = [i for i in range(len(group_A)) if i not in set(odd)]
        out = [None] * len(group_A)
        if rest:
            for i, c in zip(rest, lego_group_gemm_fn([group_A[i] for i in rest], [group_B[i] for i in rest])):
                out[i] = c
        for i in odd:
            out[i] = matmul(group_A[i], group_B[i])
        return out
    groups = len(group_A)
    group_C, sizes = [], []
    for a, b in zip(group_A, group_B):
        M, K = a.shape
        N = b.shape[1]
        group_C.append(torch.empty((M, N), device=a.device, dtype=a.dtype))
        sizes += [M, N, K]
    arr = ctypes.c_void_p * groups
    pa = arr(*[t.data_ptr() for t in group_A])
    pb = arr(*[t.data_ptr() for t in group_B])
    pc = arr(*[t.data_ptr() for t in group_C])
    sz = (ctypes.c_int * (3 * groups))(*sizes)
    runtime.call("lego_hip_grouped_gemm_f16", pa, pb, pc, sz, groups, _stream())
    return group_C


def needleman_wunsch(reference: torch.Tensor, matrix: torch.Tensor, penalty: int) -> torch.Tensor:
    """Fills the ``(n+1) x (n+1)`` int32 score ``matrix`` in place (its first row and column are the
    borders) from the substitution scores ``reference``; returns ``matrix``.  The reference's
    benchmark is a whole program (benchmarks/cuda/nw/needle.cu:165-260) with no host callable."""
    _check(reference, torch.int32, "reference")
    _check(matrix, torch.int32, "matrix")
    if reference.shape != matrix.shape or matrix.shape[0] != matrix.shape[1]:
        raise ValueError("reference and matrix must be square and of the same shape")
    runtime.call("lego_hip_nw_i32", _ptr(reference), _ptr(matrix), matrix.shape[0] - 1, int(penalty), _stream())
    return matrix


def _stencil(entry, x, c, radius, bricks, out):
    _check(x, torch.float32, "x", ndim=3)
    _check(c, torch.float32, "c", ndim=c.dim())
    n = x.shape[0]
    if x.shape != (n, n, n):
        raise ValueError("x must be a cube")
    if out is None:
        out = torch.zeros_like(x)
    else:
        _check(out, torch.float32, "out", ndim=3)
        if out.shape != x.shape or out.device != x.device:
            raise ValueError("out must have the shape and device of x")
        if out.data_ptr() == x.data_ptr():
            raise ValueError("out must not alias x")
    runtime.call(entry, _ptr(x), _ptr(out), _ptr(c), n, int(radius), 1 if bricks else 0, _stream())
    return out


def stencil_f3d(x, c, radius=1, bricks=False, out=None):
    """Dense ``(2*radius+1)^3`` stencil with the ``8 x 8 x 8`` coefficient cube ``c``; ``x`` holds the
    ``n^3`` points row-major, or brick by brick when ``bricks`` is set (``x.view(-1)`` is the
    storage either way).  Boundary points keep the value of ``out`` (zeros by default, as the
    reference program's ``cudaMemset``, benchmarks/cuda/bricks/main_tmp.cu:160-163)."""
    if c.shape != (8, 8, 8):
        raise ValueError("c must be 8 x 8 x 8")
    return _stencil("lego_hip_stencil_f3d_f32", x, c, radius, bricks, out)


def stencil_laplacian(x, c, radius=1, bricks=False, out=None):
    """Star stencil ``c[0]*x + sum_a c[a]*(six neighbours at distance a)``; ``c`` has at least
    ``radius + 1`` entries."""
    if c.dim() != 1 or c.shape[0] < radius + 1:
        raise ValueError("c must hold radius + 1 coefficients")
    return _stencil("lego_hip_stencil_laplacian_f32", x, c, radius, bricks, out)


def lud(m: torch.Tensor) -> torch.Tensor:
    """LU decomposition without pivoting, in place; returns ``m`` holding L below the diagonal
    (unit diagonal implied) and U on and above it (benchmarks/cuda/lud/lud.cu: a whole program,
    no host callable)."""
    _check(m, torch.float32, "m")
    if m.shape[0] != m.shape[1]:
        raise ValueError("m must be square")
    runtime.call("lego_hip_lud_f32", _ptr(m), m.shape[0], _stream())
    return m
