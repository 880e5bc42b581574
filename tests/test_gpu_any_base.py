"""Tensors whose base is only element aligned -- a view that starts a few elements into a buffer, such as `t[1:]`
of a tensor with an odd number of columns -- through the C ABI against the CPU oracle.  The reference's Triton
kernels take any pointer (triton_generated/softmax/softmax.py:97-160, layernorm/layernorm.py:279-307); here such
tensors take the kernels for rows and shapes of any length, which place their 16-byte accesses where the RESULT has
its 16-byte boundaries.  Inputs and results are offset independently, and guard elements around every result check
that nothing outside it is written."""
import ctypes

import pytest
import torch

from oracle import kernels as ok

pytestmark = pytest.mark.gpu
GUARD = 64


@pytest.fixture(scope="module")
def runtime():
    from lego_amd import runtime
    runtime.load_library()
    assert torch.cuda.is_available()
    return runtime


def _gen(seed):
    return torch.Generator().manual_seed(seed)


def _p(t):
    return ctypes.c_void_p(t.data_ptr())


def _view(host, offset):
    """`host` on the device as a view that starts `offset` elements into a 16-byte aligned buffer."""
    buf = torch.empty(host.numel() + offset + 8, dtype=host.dtype, device="cuda")
    view = buf[offset:offset + host.numel()].view(host.shape)
    view.copy_(host)
    assert view.data_ptr() % 16 == (offset * host.element_size()) % 16 and view.is_contiguous()
    return view


def _result(shape, dtype, offset):
    """A result tensor `offset` elements into a buffer filled with a sentinel; returns (view, check) where check()
    asserts the elements around the view still hold the sentinel."""
    n = 1
    for d in shape:
        n *= d
    buf = torch.full((n + 2 * GUARD + offset,), 7.0, dtype=dtype, device="cuda")
    view = buf[GUARD + offset:GUARD + offset + n].view(shape)

    def untouched():
        assert (buf[:GUARD + offset] == 7.0).all() and (buf[GUARD + offset + n:] == 7.0).all(), "wrote outside the result"
    return view, untouched


@pytest.mark.parametrize("dtype,rows,cols,off_in,off_out", [
    (torch.float16, 781, 1823, 1, 0),       # x[1:]-style view into an aligned result (what torch.empty hands out)
    (torch.float16, 1024, 2048, 3, 5),      # whole tiles, both bases off
    (torch.float16, 8200, 8201, 1, 7),      # the larger macro tile (from 64 Mi elements on)
    (torch.float16, 64, 96, 5, 2),          # tiny: one element per access
    (torch.float32, 1001, 999, 1, 0), (torch.float32, 2048, 1024, 2, 3), (torch.float32, 8197, 8199, 3, 1),
    (torch.float32, 7, 5, 1, 1)])
def test_transpose_of_views(runtime, dtype, rows, cols, off_in, off_out):
    print(f"transpose of a view {dtype} {rows}x{cols} +{off_in} -> +{off_out}", flush=True)
    x = (torch.rand(rows, cols, generator=_gen(1)) * 2 - 1).to(dtype)
    xd = _view(x, off_in)
    out, untouched = _result((cols, rows), dtype, off_out)
    runtime.call("lego_hip_transpose_f32" if dtype == torch.float32 else "lego_hip_transpose_f16", _p(xd), _p(out), rows, cols, None)
    torch.cuda.synchronize()
    assert torch.equal(out.cpu(), ok.transpose(x, 1, 1))
    untouched()


ROW_SHAPES = [(33, 100), (129, 781), (300, 1024), (64, 2050), (1151, 8192), (520, 8191), (70, 20001), (40, 32768),
              (4100, 8200), (9000, 1001)]      # the last two: the walking launches (tall matrices)


@pytest.mark.parametrize("dtype,tag,esz", [(torch.float16, "f16", 2), (torch.bfloat16, "bf16", 2), (torch.float32, "f32", 4)])
@pytest.mark.parametrize("M,N", ROW_SHAPES)
def test_softmax_of_views(runtime, dtype, tag, esz, M, N):
    print(f"softmax of a view {tag} {M}x{N}", flush=True)
    x = (2.0 * torch.randn(M, N, generator=_gen(2))).to(dtype)
    for off_in, off_out in ((1, 0), (3, 5)):
        xd = _view(x, off_in)
        y, untouched = _result((M, N), dtype, off_out)
        runtime.call(f"lego_hip_softmax_{tag}", _p(xd), _p(y), M, N, None)
        torch.cuda.synchronize()
        tol = 1e-6 if dtype == torch.float32 else 2e-3 if dtype == torch.float16 else 2.0 ** -9 + 1e-6     # bf16: half a spacing below 1
        assert (y.cpu().float() - ok.softmax(x).float()).abs().max().item() <= tol
        untouched()


def test_softmax_of_a_long_row_view(runtime):
    """Rows above 32768 elements (read twice) at an odd element."""
    print("softmax of a view, rows of 50257", flush=True)
    M, N = 9, 50257
    x = (2.0 * torch.randn(M, N, generator=_gen(3))).half()
    xd = _view(x, 5)
    y, untouched = _result((M, N), torch.float16, 2)
    runtime.call("lego_hip_softmax_f16", _p(xd), _p(y), M, N, None)
    torch.cuda.synchronize()
    assert (y.cpu().float() - ok.softmax(x).float()).abs().max().item() <= 2e-3
    untouched()


TYPES = [(torch.float16, "f16", 2), (torch.bfloat16, "bf16", 2), (torch.float32, "f32", 4)]
BWD_SHAPES = [(33, 100), (129, 781), (300, 1024), (64, 2050), (1151, 8192), (520, 8191), (70, 16384), (40, 20001), (33, 32768),
              (4100, 4096), (9000, 1001)]


def _rows_within_64_kib(shapes):
    """(dtype, tag, M, N) for every element type and shape whose row stays within the reference's 64 KiB."""
    return [(dtype, tag, M, N) for dtype, tag, esz in TYPES for M, N in shapes if N * esz <= 65536]


@pytest.mark.parametrize("dtype,tag,M,N", _rows_within_64_kib(ROW_SHAPES))
def test_layernorm_forward_of_views(runtime, dtype, tag, M, N):
    print(f"layernorm forward of a view {tag} {M}x{N}", flush=True)
    g = _gen(4)
    x = (2.0 * torch.randn(M, N, generator=g)).to(dtype)
    w = (1 + 0.1 * torch.randn(N, generator=g)).to(dtype)
    b = (0.1 * torch.randn(N, generator=g)).to(dtype)
    want_y, want_mean, want_rstd = ok.layernorm_fwd(x, w, b, 1e-5)
    y32 = ok.layernorm_fwd_unrounded(x, w, b, 1e-5)
    for off_x, off_y, off_w in ((1, 0, 0), (3, 5, 1)):
        xd, wd, bd = _view(x, off_x), _view(w, off_w), _view(b, off_w + 2)
        y, untouched = _result((M, N), dtype, off_y)
        mean, rstd = torch.empty(M, device="cuda"), torch.empty(M, device="cuda")
        runtime.call(f"lego_hip_layernorm_fwd_{tag}", _p(xd), _p(y), _p(wd), _p(bd), _p(mean), _p(rstd), M, N,
                     ctypes.c_float(1e-5), None)
        torch.cuda.synchronize()
        err = (y.cpu().float() - y32).abs()
        slack = (ok.half_spacing(y32, dtype) if dtype != torch.float32 else 0) + (1e-4 if dtype != torch.float32 else 2e-5)
        assert (err - slack).max().item() <= 0
        assert torch.allclose(mean.cpu(), want_mean, atol=1e-4, rtol=1e-4) and torch.allclose(rstd.cpu(), want_rstd, atol=1e-4, rtol=1e-3)
        untouched()


@pytest.mark.parametrize("dtype,tag,M,N", _rows_within_64_kib(BWD_SHAPES))
def test_layernorm_backward_of_views(runtime, dtype, tag, M, N):
    """dy, x, w and dx each at their own element offset, against fp32 autograd on the CPU."""
    print(f"layernorm backward of views {tag} {M}x{N}", flush=True)
    g = _gen(5)
    x = (2.0 * torch.randn(M, N, generator=g)).to(dtype)
    w = (1 + 0.1 * torch.randn(N, generator=g)).to(dtype)
    b = (0.1 * torch.randn(N, generator=g)).to(dtype)
    dy = (0.1 * torch.randn(M, N, generator=g)).to(dtype)
    xf, wf = x.float().requires_grad_(True), w.float().requires_grad_(True)
    bf = b.float().requires_grad_(True)
    torch.nn.functional.layer_norm(xf, (N,), wf, bf, 1e-5).backward(dy.float())
    _, mean_c, rstd_c = ok.layernorm_fwd(x, w, b, 1e-5)
    mean, rstd = mean_c.cuda(), rstd_c.cuda()
    suffix = "" if tag == "f16" else f"_{tag}"
    need = ctypes.c_ulonglong(0)
    runtime.call(f"lego_hip_layernorm_bwd{suffix}_workspace_bytes", M, N, ctypes.byref(need))
    ws = torch.full((need.value // 4,), float("nan"), device="cuda")
    for off_dy, off_x, off_w, off_dx in ((0, 1, 0, 0), (3, 1, 5, 2)):
        dyd, xd, wd = _view(dy, off_dy), _view(x, off_x), _view(w, off_w)
        dx, untouched = _result((M, N), dtype, off_dx)
        dw, dw_ok = _result((N,), dtype, 1)
        db, db_ok = _result((N,), dtype, 3)
        runtime.call(f"lego_hip_layernorm_bwd_{tag}", _p(dyd), _p(xd), _p(wd), _p(mean), _p(rstd), _p(dx), _p(dw), _p(db),
                     _p(ws), need, M, N, None)
        torch.cuda.synchronize()
        tol = {torch.float16: 2e-3, torch.bfloat16: 1.6e-2, torch.float32: 1e-4}[dtype]
        assert (dx.cpu().float() - xf.grad).abs().max().item() <= tol
        scale = max(1.0, wf.grad.abs().max().item())
        assert (dw.cpu().float() - wf.grad).abs().max().item() <= (1e-2 if dtype != torch.float32 else 1e-3) * scale
        assert (db.cpu().float() - bf.grad).abs().max().item() <= (1e-2 if dtype != torch.float32 else 1e-3) * max(1.0, bf.grad.abs().max().item())
        untouched(); dw_ok(); db_ok()
