"""GPU parity tests: the HIP path, called through the C ABI, against the CPU oracle."""
import math

import pytest
import torch

from oracle import kernels as ok

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ops():
    from lego_amd import ops, runtime
    runtime.load_library()   # fails loudly when liblego_hip.so was not built
    assert torch.cuda.is_available()
    return ops


def _gen(seed):
    return torch.Generator().manual_seed(seed)


# ---- transpose: bit exact ---------------------------------------------------------------

@pytest.mark.parametrize("dtype,rows,cols", [
    (torch.float32, 64, 64), (torch.float32, 128, 320), (torch.float32, 1024, 512), (torch.float32, 32, 256),
    (torch.float32, 96, 768), (torch.float16, 64, 64), (torch.float16, 192, 128), (torch.float16, 512, 1024),
    (torch.float16, 64, 256), (torch.float16, 320, 768),
    (torch.float32, 2048, 1024), (torch.float32, 4096, 3072),    # windowed cache-resident fp32 tiling
    (torch.float16, 8192, 2048),                    # one window of the windowed tile order
    (torch.float16, 4096, 6144), (torch.float16, 12288, 2048),    # windows of 64 x 8 macro tiles: one, and three by one
    (torch.float16, 2048, 4096), (torch.float16, 6144, 2048),     # windows of 32 x 8: one by two, three by one
    (torch.float16, 1088, 2304), (torch.float32, 1056, 2304),     # the wide tiles in skewed order (from 2 Mi elements on)
])
def test_transpose_matches_oracle(ops, dtype, rows, cols):
    print(f"transpose {dtype} {rows}x{cols}", flush=True)
    x = (torch.rand(rows, cols, generator=_gen(0)) * 2 - 1).to(dtype)
    want = ok.transpose(x, 32, 32)                 # index-array scatter through the two layouts
    assert torch.equal(want, x.t().contiguous())   # and that is the textbook transpose
    got = ops.transpose(x.cuda()).cpu()
    assert torch.equal(got, want)


def test_transpose_config1_fp32_4096(ops):
    print("transpose config 1", flush=True)
    x = torch.rand(4096, 4096, generator=_gen(0), dtype=torch.float32) * 2 - 1
    got = ops.transpose(x.cuda()).cpu()
    assert torch.equal(got, ok.transpose(x, 32, 32))


def test_transpose_config2_fp16_16384_properties(ops):
    """Full size: transposing twice is the identity and the result equals the strided view."""
    print("transpose config 2", flush=True)
    xc = torch.randn(16384, 16384, generator=_gen(1)).half()
    x = xc.cuda()
    y = ops.transpose(x)
    assert torch.equal(y, x.t())
    assert torch.equal(ops.transpose(y), x)
    # and against the CPU path itself on two strips of the matrix: the oracle's index scatter through both
    # TileBy([.., ..], [64, 64]) layouts on columns 0..255 (rows 0..255 of the result) and the last 256 columns
    for cols in (slice(0, 256), slice(16384 - 256, 16384)):
        assert torch.equal(y[cols].cpu(), ok.transpose(xc[:, cols].contiguous(), 64, 64))


def test_transpose_windowed_order_rectangular(ops):
    """Several windows per side, more across than down: a mix-up of the window digits
    would move tiles."""
    print("transpose fp16 16384x6144 (windowed order)", flush=True)
    x = torch.randn(16384, 6144, generator=_gen(2)).half().cuda()
    y = ops.transpose(x)
    assert y.shape == (6144, 16384)
    assert torch.equal(y, x.t())


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.int32, torch.int16])
def test_transpose_moves_bits_of_any_2_or_4_byte_type(ops, dtype):
    print(f"transpose {dtype}", flush=True)
    x = torch.randint(-30000, 30000, (192, 256), generator=_gen(3)).to(dtype).cuda()
    assert torch.equal(ops.transpose(x), x.t().contiguous())


@pytest.mark.parametrize("dtype,rows,cols", [(torch.float32, 100, 64), (torch.float32, 32, 64), (torch.float32, 1, 1),
                                             (torch.float16, 1823, 781), (torch.float16, 65, 4097), (torch.float32, 777, 3),
                                             (torch.float16, 8, 8), (torch.float16, 72, 264), (torch.float16, 1000, 520),
                                             (torch.float16, 4104, 1096), (torch.float16, 64, 8), (torch.float16, 8, 1024),
                                             (torch.float32, 4, 4), (torch.float32, 36, 260), (torch.float32, 1004, 516),
                                             (torch.float32, 2052, 4100),
                                             # rows that start at any element: vectors at their own alignment, the ones
                                             # that an edge cuts element by element
                                             (torch.float16, 9, 9), (torch.float16, 1001, 999), (torch.float16, 130, 257),
                                             (torch.float16, 2055, 1031), (torch.float16, 15, 4099), (torch.float16, 4099, 15),
                                             (torch.float16, 1000, 777), (torch.float16, 777, 1000), (torch.float16, 7, 300),
                                             (torch.float32, 5, 7), (torch.float32, 1001, 999), (torch.float32, 130, 257),
                                             (torch.float32, 2051, 1033), (torch.float32, 516, 1001), (torch.float32, 1001, 516),
                                             (torch.float16, 2055, 2061), (torch.float16, 15, 300001), (torch.float16, 300001, 15),
                                             (torch.float16, 4100, 1031), (torch.float16, 1031, 4100),
                                             (torch.float32, 1449, 1451), (torch.float32, 5, 500001), (torch.float32, 500001, 5),
                                             (torch.float32, 2052, 1031),
                                             # the larger macro tile, from 64 Mi elements on
                                             (torch.float16, 8200, 8201), (torch.float32, 8197, 8199),
                                             # whole vectors, from 32 Mi elements on: the wide tile with edge tests, rows
                                             # in cut and in whole 64-byte blocks (plain and non-temporal stores)
                                             (torch.float16, 8200, 4104), (torch.float16, 8224, 4128),
                                             (torch.float32, 8196, 4100), (torch.float32, 8208, 4112)])
def test_transpose_of_any_shape(ops, dtype, rows, cols):
    """Shapes no tiling divides: in whole 16-byte vectors both ways they take the wide tile with edge
    tests, otherwise 64x64 tiles (a larger tile from 64 Mi elements on) with vectors at any element, and the
    one-element-per-access kernel when a side is shorter than a vector or the matrix is tiny."""
    print(f"transpose (any shape) {dtype} {rows}x{cols}", flush=True)
    x = (torch.rand(rows, cols, generator=_gen(4)) * 2 - 1).to(dtype)
    want = ok.transpose(x, 1, 1)
    assert torch.equal(want, x.t().contiguous())
    buf = torch.full((rows * cols + 2048,), 7.0, dtype=dtype, device="cuda")
    out = buf[1024:1024 + rows * cols].view(cols, rows)
    from lego_amd import runtime
    import ctypes
    xd = x.cuda()
    runtime.call("lego_hip_transpose_f32" if dtype == torch.float32 else "lego_hip_transpose_f16",
                 ctypes.c_void_p(xd.data_ptr()), ctypes.c_void_p(out.data_ptr()), rows, cols, None)
    torch.cuda.synchronize()
    assert torch.equal(out.cpu(), want)
    assert (buf[:1024] == 7.0).all() and (buf[1024 + rows * cols:] == 7.0).all()       # nothing outside the matrix was written


def test_transpose_offsets_beyond_32_bits(ops):
    """More than 2^32 elements: the first and the last rows and columns of the result are compared."""
    print("transpose of more than 2^32 elements", flush=True)
    rows, cols = 65536 + 64, 65536
    x = torch.empty(rows, cols, device="cuda", dtype=torch.half).normal_(generator=torch.Generator(device="cuda").manual_seed(28))
    y = ops.transpose(x)
    assert y.shape == (cols, rows)
    for r in (slice(0, 64), slice(rows - 64, rows)):
        assert torch.equal(y[:, r], x[r, :].t())
    for c in (slice(0, 64), slice(cols - 64, cols)):
        assert torch.equal(y[c, :], x[:, c].t())


def test_transpose_rejects_bad_arguments(ops):
    from lego_amd.runtime import LegoHipError
    with pytest.raises(ValueError):
        ops.transpose(torch.zeros(64, 64, device="cuda").t())
    with pytest.raises(LegoHipError):
        x = torch.zeros(64, 64, device="cuda")
        from lego_amd import runtime
        import ctypes
        runtime.call("lego_hip_transpose_f32", ctypes.c_void_p(x.data_ptr()), ctypes.c_void_p(x.data_ptr()), 64, 64, None)


# ---- softmax / layernorm: max abs err <= 2e-3 ------------------------------------------------

TOL = 2e-3


def _assert_layernorm_forward(y, x, w, b, eps=1e-5):
    """A 16-bit LayerNorm result against the un-rounded fp32 oracle.  The contract is on the fp32
    arithmetic (max abs err <= 2e-3 after fp32 accumulation); the store then rounds to 16 bits, which
    moves a value by up to half a spacing (2^-10 for fp16 values in [2, 4)).  So: the result is within
    half a spacing of the fp32 oracle, plus 1e-4 for the fp32 arithmetic itself (summation order), and
    wherever |y| < 2 the literal bound holds against the rounded oracle as well."""
    ref32 = ok.layernorm_fwd_unrounded(x, w, b, eps)
    err = (y.cpu().float() - ref32).abs()
    slack = ok.half_spacing(ref32, x.dtype) + 1e-4
    worst = (err - slack).max().item()
    assert worst <= 0, f"{worst:.3e} beyond half a spacing + 1e-4"
    small = ref32.abs() < 2
    if x.dtype == torch.float16 and small.any():
        assert (y.cpu().float() - ref32.to(x.dtype).float()).abs()[small].max().item() <= TOL


@pytest.mark.parametrize("wpr", [None, 1, 2, 4, 8])
@pytest.mark.parametrize("M,N", [(7, 8), (33, 520), (64, 1024), (5, 2048), (129, 4096), (16, 8192), (3, 16384),
                                 (4100, 8200),      # tall and long: the default takes teams of eight waves
                                 (2500, 3080),      # one round of workgroups: the default takes teams of two
                                 (16390, 1600)])    # very tall, four vectors per lane of one wave: teams of two as well
def test_softmax_matches_oracle(ops, M, N, wpr):
    print(f"softmax {M}x{N} wpr={wpr}", flush=True)
    if wpr is not None and N > min(8192 * wpr, 16384):
        from lego_amd.runtime import LegoHipError
        with pytest.raises(LegoHipError):      # a row must fit the registers of its team
            ops.softmax(torch.zeros(M, N, device="cuda", dtype=torch.half), waves_per_row=wpr)
        return
    x = (2.0 * torch.randn(M, N, generator=_gen(2))).half()
    want = ok.softmax(x)
    got = ops.softmax(x.cuda(), waves_per_row=wpr).cpu()
    assert (got.float() - want.float()).abs().max().item() <= TOL
    assert torch.allclose(got.float().sum(-1), torch.ones(M), atol=2e-2)


@pytest.mark.parametrize("dtype", [torch.float16, torch.float32])
@pytest.mark.parametrize("M,N", [(3, 32776), (2, 50257), (5, 65536), (2, 131072), (1, 200003)])
def test_softmax_rows_read_twice(ops, dtype, M, N):
    """Rows above 32768 elements (vocabulary-sized rows among them): running maximum and sum, then
    a second pass."""
    print(f"softmax long rows {dtype} {M}x{N}", flush=True)
    x = (2.0 * torch.randn(M, N, generator=_gen(24))).to(dtype)
    x[0, 7] = 11.0               # a maximum that arrives early ...
    x[-1, N - 3] = 12.5          # ... and one that arrives late
    want = ok.softmax(x)
    got = ops.softmax(x.cuda()).cpu()
    assert (got.float() - want.float()).abs().max().item() <= (TOL if dtype == torch.float16 else 1e-6)
    assert torch.allclose(got.float().sum(-1), torch.ones(M), atol=2e-2 if dtype == torch.float16 else 1e-4)


def test_softmax_reference_test_shape_fp32(ops):
    """The reference's own check (softmax.py:237-241): seed 0, x = randn(1823, 781) in fp32,
    compared with torch.softmax at allclose's default tolerance."""
    print("softmax fp32 1823x781", flush=True)
    torch.manual_seed(0)
    x = torch.randn(1823, 781)
    got = ops.softmax(x.cuda()).cpu()
    assert torch.allclose(got, torch.softmax(x, dim=1))
    assert (got - ok.softmax(x)).abs().max().item() <= 1e-6


@pytest.mark.parametrize("dtype", [torch.float16, torch.float32])
@pytest.mark.parametrize("M,N", [(5, 1), (9, 3), (17, 781), (4, 1000), (3, 4099), (2, 16383), (6, 2048), (3, 16384),
                                 (3, 16392), (2, 20001), (5, 32767), (4, 32768),
                                 # tall and ragged: teams walk rows that start alike, the next row's loads in flight
                                 (8300, 781), (8195, 250), (8200, 1001), (2050, 4099), (2049, 8191), (2300, 2050),
                                 (1030, 12001), (1100, 16383), (515, 20001), (600, 32767),
                                 # tall, rows of 12-32 KiB: teams of eight waves in fp32 as well
                                 (4100, 4096), (4097, 8192), (4096, 3076),
                                 # ... and for 16-bit rows of any length
                                 (4100, 8191), (4097, 12001), (4100, 4099)])
def test_softmax_ragged_and_fp32(ops, dtype, M, N):
    print(f"softmax {dtype} {M}x{N}", flush=True)
    x = (2.0 * torch.randn(M, N, generator=_gen(2))).to(dtype)
    want = ok.softmax(x)
    got = ops.softmax(x.cuda()).cpu()
    assert (got.float() - want.float()).abs().max().item() <= (TOL if dtype == torch.float16 else 1e-6)


@pytest.mark.parametrize("dtype", [torch.float16, torch.float32])
@pytest.mark.parametrize("M,N", [(5, 1), (9, 3), (17, 781), (3, 4099), (6, 2048), (3, 16384), (3, 16392), (2, 20001),
                                 (4, 32768),
                                 # tall and ragged: teams walk rows that start alike, gamma and beta shifted into LDS
                                 (8300, 781), (8195, 250), (8200, 1001), (2050, 4099), (2049, 8191), (2300, 2050),
                                 (515, 20001), (600, 32767), (1030, 12001), (1100, 16383), (4100, 3001),
                                 # tall, rows of 12-32 KiB: teams of eight waves in fp32 as well (gamma and beta in LDS)
                                 (4100, 4096), (4097, 8192), (4096, 3076),
                                 # ... and for 16-bit rows of any length
                                 (4100, 8191), (4097, 12001), (4100, 4099)])
def test_layernorm_ragged_and_fp32(ops, dtype, M, N):
    print(f"layernorm {dtype} {M}x{N}", flush=True)
    if N * torch.empty((), dtype=dtype).element_size() > 65536:
        with pytest.raises(RuntimeError, match="64KB"):    # the reference's limit and message (layernorm.py:293-294)
            ops.layer_norm_fwd(torch.zeros(M, N, dtype=dtype, device="cuda"), torch.zeros(N, dtype=dtype, device="cuda"),
                               torch.zeros(N, dtype=dtype, device="cuda"), 1e-5)
        return
    g = _gen(3)
    x = (2.0 * torch.randn(M, N, generator=g)).to(dtype)
    w = (1 + 0.1 * torch.randn(N, generator=g)).to(dtype)
    b = (0.1 * torch.randn(N, generator=g)).to(dtype)
    want_y, want_mean, want_rstd = ok.layernorm_fwd(x, w, b, 1e-5)
    y, mean, rstd = ops.layer_norm_fwd(x.cuda(), w.cuda(), b.cuda(), 1e-5)
    if dtype == torch.float16:
        _assert_layernorm_forward(y, x, w, b)
    else:
        assert (y.cpu().float() - want_y.float()).abs().max().item() <= 2e-5
    assert torch.allclose(mean.cpu(), want_mean, atol=1e-4, rtol=1e-4)
    if N > 1:
        assert torch.allclose(rstd.cpu(), want_rstd, atol=1e-4, rtol=1e-3)


@pytest.mark.parametrize("M,N", [(24600, 8191), (201500, 1001), (16386, 8191), (65541, 781), (33000, 6152)])
def test_rows_of_any_length_in_several_launches(ops, M, N):
    """Tall matrices of rows of any length: the walking kernels run in launches of about 16 rows per team (64 for rows
    of whole vectors), one after the other, equal in length, and a remainder of under a quarter of a launch is folded
    into the launches before it (16386 x 8191: launches of 8704 and 7682 rows; 65541 x 781: one launch of 17 steps;
    33000 x 6152, rows of whole vectors: one launch of 65 steps).  At this size:
    row sums of the softmax, the statistics against torch on the GPU, and the first and last rows (the ends of
    the first and of the last launch) against the oracle."""
    print(f"rows of any length, large result {M}x{N}", flush=True)
    g = _gen(61)
    xd = (2.0 * torch.randn(M, N, generator=g, dtype=torch.float32)).half().cuda()
    w = (1 + 0.1 * torch.randn(N, generator=g)).half()
    b = (0.1 * torch.randn(N, generator=g)).half()
    sm = ops.softmax(xd)
    assert (sm.float().sum(-1) - 1).abs().max().item() <= 2e-2
    y, mean, rstd = ops.layer_norm_fwd(xd, w.cuda(), b.cuda(), 1e-5)
    xf = xd.float()
    assert (mean - xf.mean(-1)).abs().max().item() <= 1e-4
    assert ((rstd - torch.rsqrt(xf.var(-1, unbiased=False) + 1e-5)).abs() <= 1e-3 * rstd.abs()).all()
    del xf
    for rows in (slice(0, 48), slice(M // 2 - 24, M // 2 + 24), slice(M - 48, M), slice(8704 - 24, 8704 + 24)):
        x = xd[rows].cpu()
        assert (sm[rows].cpu().float() - ok.softmax(x).float()).abs().max().item() <= TOL
        _assert_layernorm_forward(y[rows], x, w, b)


@pytest.mark.parametrize("N", [16392, 30001, 32768])
def test_layernorm_fp32_long_rows_through_the_c_abi(ops, N):
    """fp32 rows above 64 KiB: the Python wrapper keeps the reference's limit, the library takes them."""
    import ctypes
    from lego_amd import runtime
    print(f"layernorm fp32 long row {N}", flush=True)
    M = 5
    g = _gen(23)
    x = 2.0 * torch.randn(M, N, generator=g)
    w = 1 + 0.1 * torch.randn(N, generator=g)
    b = 0.1 * torch.randn(N, generator=g)
    want_y, want_mean, want_rstd = ok.layernorm_fwd(x, w, b, 1e-5)
    xd, wd, bd = x.cuda(), w.cuda(), b.cuda()
    y = torch.empty_like(xd)
    mean = torch.empty(M, device="cuda")
    rstd = torch.empty(M, device="cuda")
    p = lambda t: ctypes.c_void_p(t.data_ptr())
    runtime.call("lego_hip_layernorm_fwd_f32", p(xd), p(y), p(wd), p(bd), p(mean), p(rstd), M, N, 1e-5, None)
    torch.cuda.synchronize()
    assert (y.cpu() - want_y).abs().max().item() <= 2e-5
    assert torch.allclose(mean.cpu(), want_mean, atol=1e-4, rtol=1e-4)
    assert torch.allclose(rstd.cpu(), want_rstd, atol=1e-4, rtol=1e-3)


@pytest.mark.parametrize("wpr", [None, 1, 2, 4, 8])
# 1151 and 4100 rows with eight waves: workgroups that stage gamma and beta in LDS and walk two to nine rows each
# 600 and 515 rows of more than 16384 elements: the same walk with sixteen waves, one row across 1024 lanes
@pytest.mark.parametrize("M,N", [(7, 8), (33, 520), (64, 1024), (129, 4096), (1151, 8192), (3, 16384), (4100, 8200),
                                 (1030, 16384), (600, 32768), (515, 20488), (511, 32768),
                                 (2500, 3080),      # one round of workgroups: the default takes teams of two waves
                                 # teams of four waves with four vectors per lane walk rows as well (from 2048 rows on)
                                 (2050, 5128), (2049, 8192),
                                 (16390, 1600)])    # very tall, four vectors per lane of one wave: the default takes two waves
def test_layernorm_matches_oracle(ops, M, N, wpr):
    print(f"layernorm {M}x{N} wpr={wpr}", flush=True)
    if wpr is not None and N > min(8192 * wpr, 16384):
        from lego_amd.runtime import LegoHipError
        z = torch.zeros(M, N, device="cuda", dtype=torch.half)
        with pytest.raises(LegoHipError):      # a row must fit the registers of its team
            ops.layer_norm_fwd(z, z[0].clone(), z[0].clone(), 1e-5, waves_per_row=wpr)
        return
    g = _gen(3)
    x = (2.0 * torch.randn(M, N, generator=g)).half()
    w = (1 + 0.1 * torch.randn(N, generator=g)).half()
    b = (0.1 * torch.randn(N, generator=g)).half()
    want_y, want_mean, want_rstd = ok.layernorm_fwd(x, w, b, 1e-5)
    y, mean, rstd = ops.layer_norm_fwd(x.cuda(), w.cuda(), b.cuda(), 1e-5, waves_per_row=wpr)
    _assert_layernorm_forward(y, x, w, b)
    assert torch.allclose(mean.cpu(), want_mean, atol=1e-4, rtol=1e-4)
    assert torch.allclose(rstd.cpu(), want_rstd, atol=1e-4, rtol=1e-4)


def test_layernorm_reference_test_shape(ops):
    """The reference's own test case (layernorm.py:435-458): M=1151, N=8192, x = -2.3 + 0.5*randn,
    w, b uniform, atol=1e-2."""
    print("layernorm reference shape", flush=True)
    g = _gen(0)
    w, b = torch.rand(8192, generator=g).half(), torch.rand(8192, generator=g).half()
    x = (-2.3 + 0.5 * torch.randn(1151, 8192, generator=g)).half()
    want = torch.nn.functional.layer_norm(x.float(), (8192,), w.float(), b.float(), 1e-5).half()
    from lego_amd.ops import lego_layer_norm
    got = lego_layer_norm(x.cuda(), (8192,), w.cuda(), b.cuda(), 1e-5).cpu()
    assert torch.allclose(got.float(), want.float(), atol=1e-2, rtol=0)
    _assert_layernorm_forward(got, x, w, b)


def test_layernorm_backward_reference_test(ops):
    """The reference's forward+backward test (layernorm.py:435-458): M=1151, N=8192, fp16,
    y, dx, dw, db against torch autograd at atol=1e-2."""
    print("layernorm backward reference test", flush=True)
    from lego_amd.ops import lego_layer_norm
    torch.manual_seed(0)
    M, N = 1151, 8192
    weight = torch.rand(N, dtype=torch.float16, device="cuda", requires_grad=True)
    bias = torch.rand(N, dtype=torch.float16, device="cuda", requires_grad=True)
    x = (-2.3 + 0.5 * torch.randn(M, N, dtype=torch.float16, device="cuda"))
    dy = 0.1 * torch.randn_like(x)
    x.requires_grad_(True)
    y = lego_layer_norm(x, (N,), weight, bias, 1e-5)
    y.backward(dy, retain_graph=True)
    dx, dw, db = [t.grad.clone() for t in (x, weight, bias)]
    x.grad, weight.grad, bias.grad = None, None, None
    # the oracle: fp32 autograd on the CPU
    xc, wc, bc = (t.detach().cpu().float().requires_grad_(True) for t in (x, weight, bias))
    yr = torch.nn.functional.layer_norm(xc, (N,), wc, bc, 1e-5)
    yr.backward(dy.cpu().float())
    assert torch.allclose(y.detach().cpu().float(), yr.detach(), atol=1e-2, rtol=0)
    assert torch.allclose(dx.cpu().float(), xc.grad, atol=1e-2, rtol=0)
    assert (dx.cpu().float() - xc.grad).abs().max().item() <= TOL
    # dw, db are sums over 1151 rows: compare relative to their magnitude (fp16 output)
    assert torch.allclose(dw.cpu().float(), wc.grad, atol=1e-2, rtol=2e-3)
    assert torch.allclose(db.cpu().float(), bc.grad, atol=1e-2, rtol=2e-3)


@pytest.mark.parametrize("M,N", [(1, 8), (3, 520), (700, 1024), (513, 2048), (64, 8192), (300, 8200), (129, 15872),
                                 (40, 16384), (5, 16392), (300, 24576), (70, 32768),
                                 (3, 1), (5, 7), (17, 781), (130, 1000), (9, 4099), (4, 20001), (3, 32767),
                                 # a wavefront per row, four rows per workgroup: fewer rows than waves, a last
                                 # workgroup with one row, more rows than the 4096 teams of a full launch
                                 (2, 512), (5, 256), (4101, 504), (9000, 1024), (6, 1016),
                                 # rows of any length, more rows than workgroups: a workgroup's rows start alike and
                                 # split into head, vectors and tail at the same columns
                                 (1100, 781), (700, 1001), (1030, 2050), (600, 4099), (530, 8191), (300, 12001),
                                 (515, 16383), (520, 250), (1100, 33), (513, 7)])
def test_layernorm_backward_matches_oracle(ops, M, N):
    print(f"layernorm backward {M}x{N}", flush=True)
    g = _gen(6)
    x = (2.0 * torch.randn(M, N, generator=g)).half()
    w = (1 + 0.1 * torch.randn(N, generator=g)).half()
    b = (0.1 * torch.randn(N, generator=g)).half()
    dy = (0.1 * torch.randn(M, N, generator=g)).half()
    _, mean, rstd = ops.layer_norm_fwd(x.cuda(), w.cuda(), b.cuda(), 1e-5)
    dx, dw, db = ops.layer_norm_bwd(dy.cuda(), x.cuda(), w.cuda(), mean, rstd)
    xc, wc, bc = (t.float().requires_grad_(True) for t in (x, w, b))
    torch.nn.functional.layer_norm(xc, (N,), wc, bc, 1e-5).backward(dy.float())
    assert (dx.cpu().float() - xc.grad).abs().max().item() <= TOL
    scale = max(1.0, wc.grad.abs().max().item())
    assert (dw.cpu().float() - wc.grad).abs().max().item() <= 2e-3 * scale
    assert (db.cpu().float() - bc.grad).abs().max().item() <= 2e-3 * max(1.0, bc.grad.abs().max().item())


def test_layernorm_backward_rejects_foreign_statistics(ops):
    """mean and rstd reach the kernel as raw pointers: anything but one float32 per row on the device is refused."""
    print("layernorm backward argument checks", flush=True)
    x = torch.zeros(4, 64, dtype=torch.half, device="cuda")
    w = torch.ones(64, dtype=torch.half, device="cuda")
    good = torch.zeros(4, device="cuda")
    for mean, rstd in ((good.cpu(), good), (good, good.half()), (good[:3], good), (good, torch.zeros(8, device="cuda")[::2]),
                       (good.view(2, 2), good)):
        with pytest.raises(ValueError):
            ops.layer_norm_bwd(x, x, w, mean, rstd)
    with pytest.raises(ValueError):
        ops.layer_norm_bwd(torch.zeros(4, 32, dtype=torch.half, device="cuda"), x, w, good, good)


@pytest.mark.parametrize("M,N", [(1, 4), (7, 5), (300, 1000), (129, 4096), (33, 4099), (40, 16384),
                                 # rows in whole groups of eight take the fused kernels: a wavefront per row (512, 1016),
                                 # 256 lanes with 1, 2 and 4 groups per lane, 512 lanes; 1004 is in whole vectors only
                                 (4101, 512), (70, 1016), (600, 2048), (50, 3000), (513, 8192), (9, 12288), (30, 1004),
                                 # rows of any length through the same kernels
                                 (1100, 781), (600, 4099), (530, 8190), (300, 12001), (1030, 1003), (515, 16381)])
def test_layernorm_backward_fp32(ops, M, N):
    """fp32 tensors through the autograd wrapper, against fp64 autograd on the CPU."""
    from lego_amd.ops import lego_layer_norm
    print(f"layernorm backward fp32 {M}x{N}", flush=True)
    g = _gen(29)
    x = 2.0 * torch.randn(M, N, generator=g)
    w = 1 + 0.1 * torch.randn(N, generator=g)
    b = 0.1 * torch.randn(N, generator=g)
    dy = 0.1 * torch.randn(M, N, generator=g)
    xd, wd, bd = (t.cuda().requires_grad_(True) for t in (x, w, b))
    lego_layer_norm(xd, (N,), wd, bd, 1e-5).backward(dy.cuda())
    xc, wc, bc = (t.double().requires_grad_(True) for t in (x, w, b))
    torch.nn.functional.layer_norm(xc, (N,), wc, bc, 1e-5).backward(dy.double())
    assert (xd.grad.cpu().double() - xc.grad).abs().max().item() <= 2e-5
    assert (wd.grad.cpu().double() - wc.grad).abs().max().item() <= 2e-5 * max(1.0, wc.grad.abs().max().item())
    assert (bd.grad.cpu().double() - bc.grad).abs().max().item() <= 2e-5 * max(1.0, bc.grad.abs().max().item())


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.float32])
@pytest.mark.parametrize("M,N", [(1, 8), (37, 24), (300, 64), (77, 120), (1000, 128), (41, 136), (513, 248), (260, 256),
                                 # of any length: head and tail elements on the first lanes of the team
                                 (64, 7), (37, 25), (300, 63), (77, 121), (1000, 127), (41, 129), (513, 250), (260, 255)])
def test_short_rows_share_a_wave(ops, dtype, M, N):
    """Rows of at most 16 or 32 vectors are dealt 4 or 2 to a wave (teams of 16 or 32 lanes, 16 or 8 rows per
    workgroup, LayerNorm two rows per team): row counts that leave teams and workgroups partly empty, row
    lengths at, between and just past the team sizes of both element widths."""
    print(f"short rows {dtype} {M}x{N}", flush=True)
    g = _gen(71)
    x = (2.0 * torch.randn(M, N, generator=g)).to(dtype)
    w = (1 + 0.1 * torch.randn(N, generator=g)).to(dtype)
    b = (0.1 * torch.randn(N, generator=g)).to(dtype)
    got = ops.softmax(x.cuda()).cpu()
    tol = {torch.float16: TOL, torch.bfloat16: 2.0 ** -9 + 1e-6, torch.float32: 1e-6}[dtype]
    assert (got.float() - ok.softmax(x).float()).abs().max().item() <= tol
    assert (got.float().sum(-1) - 1).abs().max().item() <= {torch.float32: 1e-5}.get(dtype, 2e-2)
    y, mean, rstd = ops.layer_norm_fwd(x.cuda(), w.cuda(), b.cuda(), 1e-5)
    _, want_mean, want_rstd = ok.layernorm_fwd(x, w, b, 1e-5)
    assert (mean.cpu() - want_mean).abs().max().item() <= 1e-5
    assert ((rstd.cpu() - want_rstd).abs() <= 1e-4 * want_rstd.abs()).all()
    if dtype == torch.float32:
        assert (y.cpu() - ok.layernorm_fwd_unrounded(x, w, b)).abs().max().item() <= 2e-5
    else:
        _assert_layernorm_forward(y, x, w, b)


@pytest.mark.parametrize("M,N", [(5, 8), (9, 781), (33, 2048), (64, 8192), (3, 8191), (4, 20000), (2, 32768), (2, 50257),
                                 (4100, 8200), (4100, 8191)])      # tall and long: teams of eight waves
def test_softmax_bfloat16(ops, M, N):
    print(f"softmax bf16 {M}x{N}", flush=True)
    x = (2.0 * torch.randn(M, N, generator=_gen(30))).bfloat16()
    want = torch.softmax(x.float(), -1)
    got = ops.softmax(x.cuda()).cpu()
    assert got.dtype == torch.bfloat16
    # half a bfloat16 spacing of the largest possible value, 1: 2^-9
    assert (got.float() - want).abs().max().item() <= 2.0 ** -9 + 1e-6


@pytest.mark.parametrize("M,N", [(5, 8), (9, 781), (33, 2048), (64, 8192), (3, 8191), (4, 20000), (2, 32768),
                                 (4100, 8200), (530, 24576),    # tall and long: gamma and beta staged in LDS
                                 (1100, 781), (530, 8191), (260, 16383), (4100, 8191)])
def test_layernorm_bfloat16_forward_and_backward(ops, M, N):
    """bfloat16 tensors through the autograd wrapper, against fp32 autograd on the CPU."""
    from lego_amd.ops import lego_layer_norm
    print(f"layernorm bf16 {M}x{N}", flush=True)
    g = _gen(31)
    x = (2.0 * torch.randn(M, N, generator=g)).bfloat16()
    w = (1 + 0.1 * torch.randn(N, generator=g)).bfloat16()
    b = (0.1 * torch.randn(N, generator=g)).bfloat16()
    dy = (0.1 * torch.randn(M, N, generator=g)).bfloat16()
    xd, wd, bd = (t.cuda().requires_grad_(True) for t in (x, w, b))
    y = lego_layer_norm(xd, (N,), wd, bd, 1e-5)
    y.backward(dy.cuda())
    xc, wc, bc = (t.float().requires_grad_(True) for t in (x, w, b))
    yr = torch.nn.functional.layer_norm(xc, (N,), wc, bc, 1e-5)
    yr.backward(dy.float())
    # results are rounded to bfloat16: half a spacing relative to the magnitude, 2^-9
    _assert_layernorm_forward(y.detach(), x, w, b)
    assert ((xd.grad.cpu().float() - xc.grad).abs() <= 2.0 ** -8 * xc.grad.abs() + 1e-3).all()
    assert ((wd.grad.cpu().float() - wc.grad).abs() <= 2.0 ** -8 * wc.grad.abs() + 2e-3 * max(1.0, wc.grad.abs().max().item())).all()
    assert ((bd.grad.cpu().float() - bc.grad).abs() <= 2.0 ** -8 * bc.grad.abs() + 2e-3 * max(1.0, bc.grad.abs().max().item())).all()


def test_config3_full_size(ops):
    print("config 3 full size", flush=True)
    g = _gen(2)
    x = (2.0 * torch.randn(8192, 8192, generator=g)).half()
    g3 = _gen(3)
    w = (1 + 0.1 * torch.randn(8192, generator=g3)).half()
    b = (0.1 * torch.randn(8192, generator=g3)).half()
    xd = x.cuda()
    s = ops.softmax(xd).cpu()
    assert (s.float() - ok.softmax(x).float()).abs().max().item() <= TOL
    y, mean, rstd = ops.layer_norm_fwd(xd, w.cuda(), b.cuda(), 1e-5)
    want_y, want_mean, want_rstd = ok.layernorm_fwd(x, w, b, 1e-5)
    _assert_layernorm_forward(y, x, w, b)
    assert torch.allclose(mean.cpu(), want_mean, atol=1e-4, rtol=1e-4)


# ---- GEMM: relative error <= 1e-2 against fp32 accumulation ------------------------------------

def _rel_err(got, want):
    return ((got.float() - want.float()).norm() / want.float().norm()).item()


@pytest.mark.parametrize("M,N,K", [(256, 256, 64), (256, 256, 512), (512, 256, 128), (256, 768, 256),
                                   (1024, 1024, 1024), (3072, 512, 320)])
def test_gemm_matches_oracle(ops, M, N, K):
    print(f"gemm {M}x{N}x{K}", flush=True)
    g = _gen(4)
    a = (torch.randn(M, K, generator=g) / math.sqrt(K)).half()
    b = (torch.randn(K, N, generator=g) / math.sqrt(K)).half()
    want = ok.gemm(a, b)
    got = ops.matmul(a.cuda(), b.cuda()).cpu()
    assert _rel_err(got, want) <= 1e-2
    assert (got.float() - want.float()).abs().max().item() <= 1e-2   # the reference's own atol


def test_gemm_integer_exact(ops):
    """Small-integer operands make every partial sum exact in fp32 and fp16: any indexing
    mistake (a transposed tile, a wrong k block) changes the integers."""
    print("gemm integer exact", flush=True)
    g = _gen(7)
    a = torch.randint(-2, 3, (512, 256), generator=g).half()
    b = torch.randint(-2, 3, (256, 768), generator=g).half()
    want = (a.double() @ b.double())
    got = ops.matmul(a.cuda(), b.cuda()).cpu()
    assert torch.equal(got.double(), want)


@pytest.mark.parametrize("M,N,K", [(256, 256, 64), (300, 264, 72), (1000, 520, 136), (512, 768, 256)])
def test_gemm_on_32x32x16_mfmas_is_exact_on_small_integers(ops, M, N, K):
    """The build of the 256 x 256-tile kernel on the 32x32x16 MFMA (taken by launches that leave many CUs without a
    tile), through its tuning entry point: whole and ragged tiles, a ragged last k-tile, bit for bit."""
    print(f"gemm on 32x32x16 MFMAs {M}x{N}x{K}", flush=True)
    import ctypes
    from lego_amd import runtime
    g = _gen(71)
    a = torch.randint(-2, 3, (M, K), generator=g).half()
    b = torch.randint(-2, 3, (K, N), generator=g).half()
    ad, bd = a.cuda(), b.cuda()
    c = torch.full((M, N), float("nan"), dtype=torch.half, device="cuda")
    p = lambda t: ctypes.c_void_p(t.data_ptr())
    runtime.call("lego_hip_gemm_f16_variant", p(ad), p(bd), p(c), M, N, K, 1, None)
    torch.cuda.synchronize()
    assert torch.equal(c.cpu().double(), a.double() @ b.double())


@pytest.mark.parametrize("M,N,K", [(2304, 4096, 64), (2300, 4088, 72), (3072, 3072, 128), (2560, 4096, 64),
                                   # a half round left over: big tiles by the estimate of the launch's time
                                   (6144, 4096, 64), (4352, 4096, 64)])
def test_gemm_launches_that_leave_cus_idle(ops, M, N, K):
    """129 to 175 tiles of 256 x 256 (one round that leaves a third of the CUs idle) take the 32x32x16 build, with
    and without the fused activation; products of one and a half rounds choose between the tile sizes by estimate.
    Small integers: bit for bit."""
    print(f"gemm sparse round {M}x{N}x{K}", flush=True)
    g = _gen(72)
    a = torch.randint(-2, 3, (M, K), generator=g).half()
    b = torch.randint(-2, 3, (K, N), generator=g).half()
    want = a.float() @ b.float()                       # |sums| <= 4 * 128: exact in fp32 and fp16
    ad, bd = a.cuda(), b.cuda()
    assert torch.equal(ops.matmul(ad, bd).cpu().float(), want)
    act = ops.matmul(ad, bd, activation="leaky_relu").cpu()
    assert torch.equal(act, torch.where(want >= 0, want, 0.01 * want).half())


@pytest.mark.parametrize("kind", ["f16", "bf16", "bf16_to_f16"])
@pytest.mark.parametrize("ta,tb", [(False, False), (False, True), (True, False), (True, True)])
@pytest.mark.parametrize("M,N,K", [(2304, 4096, 64), (2296, 4088, 72)])
def test_gemm_sparse_round_in_every_layout_and_type(ops, kind, ta, tb, M, N, K):
    """144 tiles of 256 x 256, whole and ragged: the 32x32x16 builds of all four operand layouts and the three 16-bit
    type combinations, with the fused activation.  Operands of -1, 0, 1: every sum is exact in bfloat16 too."""
    print(f"gemm sparse round {kind} ta={ta} tb={tb} {M}x{N}x{K}", flush=True)
    dtype = torch.float16 if kind == "f16" else torch.bfloat16
    out = torch.bfloat16 if kind == "bf16" else torch.float16
    g = _gen(73)
    a = torch.randint(-1, 2, (M, K), generator=g).to(dtype)
    b = torch.randint(-1, 2, (K, N), generator=g).to(dtype)
    want = a.float() @ b.float()
    ad = a.t().contiguous().cuda().t() if ta else a.cuda()
    bd = b.t().contiguous().cuda().t() if tb else b.cuda()
    assert torch.equal(ops.matmul(ad, bd, out_dtype=out).cpu().float(), want)
    act = ops.matmul(ad, bd, activation="leaky_relu", out_dtype=out).cpu()
    assert torch.equal(act, torch.where(want >= 0, want, 0.01 * want).to(out))


def test_grouped_gemm_matches_oracle(ops):
    print("grouped gemm", flush=True)
    g = _gen(5)
    shapes = [(256, 256, 64), (512, 256, 128), (256, 1024, 256), (768, 512, 192), (1024, 1024, 512)]
    A = [(torch.randn(m, k, generator=g) / math.sqrt(k)).half() for m, n, k in shapes]
    B = [(torch.randn(k, n, generator=g) / math.sqrt(k)).half() for m, n, k in shapes]
    want = ok.grouped_gemm(A, B)
    got = ops.lego_group_gemm_fn([a.cuda() for a in A], [b.cuda() for b in B])
    for c, w in zip(got, want):
        assert _rel_err(c.cpu(), w) <= 1e-2


@pytest.mark.parametrize("ta,tb", [(False, False), (False, True), (True, False), (True, True)])
@pytest.mark.parametrize("M,N,K", [(128, 128, 128), (8, 8, 64), (384, 640, 192), (1000, 264, 320), (256, 520, 64)])
def test_gemm_ragged_tiles(ops, ta, tb, M, N, K):
    """M and N in whole 16-byte chunks but not in whole 256 x 256 tiles (the reference's own
    grouped test multiplies 128 x 128 x 128, grouped_gemm.py:316-350)."""
    print(f"gemm ragged ta={ta} tb={tb} {M}x{N}x{K}", flush=True)
    g = _gen(15)
    a = (torch.randn(M, K, generator=g) / math.sqrt(K)).half()
    b = (torch.randn(K, N, generator=g) / math.sqrt(K)).half()
    want = ok.gemm(a, b)
    ad = a.t().contiguous().cuda().t() if ta else a.cuda()
    bd = b.t().contiguous().cuda().t() if tb else b.cuda()
    # the result is carved out of a larger buffer filled with a sentinel: nothing outside M x N may change
    buf = torch.full((M * N + 4096,), 7.0, dtype=torch.half, device="cuda")
    from lego_amd import runtime
    import ctypes
    runtime.call("lego_hip_gemm_f16_ex", ctypes.c_void_p(ad.t().data_ptr() if ta else ad.data_ptr()),
                 ctypes.c_void_p(bd.t().data_ptr() if tb else bd.data_ptr()), ctypes.c_void_p(buf.data_ptr()),
                 M, N, K, int(ta), int(tb), 0, None)
    torch.cuda.synchronize()
    got = buf[:M * N].view(M, N).cpu()
    assert _rel_err(got, want) <= 1e-2
    assert (got.float() - want.float()).abs().max().item() <= 1e-2
    assert (buf[M * N:] == 7.0).all()
    assert torch.equal(ops.matmul(ad, bd).cpu(), got)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float8_e5m2, torch.float8_e4m3fn])
def test_gemm_ragged_tiles_other_element_types(ops, dtype):
    M, N, K = 272, 528, 256
    print(f"gemm ragged {dtype} {M}x{N}x{K}", flush=True)
    g = _gen(17)
    a = torch.randn(M, K, generator=g).half().to(dtype)
    b = torch.randn(K, N, generator=g).half().to(dtype)
    want = a.float() @ b.float()
    for ta in (False, True):
        for tb in (False, True):
            ad = a.t().contiguous().cuda().t() if ta else a.cuda()
            bd = b.t().contiguous().cuda().t() if tb else b.cuda()
            got = ops.matmul(ad, bd).cpu().float()
            assert _rel_err(got, want) <= 1e-2, (ta, tb)


@pytest.mark.parametrize("ta,tb", [(False, False), (False, True), (True, False), (True, True)])
@pytest.mark.parametrize("M,N,K", [(3072, 3072, 128), (3080, 3000, 64)])
def test_gemm_many_tiles(ops, ta, tb, M, N, K):
    """More than 128 tiles of 256 x 256: the one-workgroup-per-CU kernel (smaller problems take
    the 128 x 128 tiles), whole and ragged."""
    print(f"gemm many tiles ta={ta} tb={tb} {M}x{N}x{K}", flush=True)
    g = _gen(18)
    a = (torch.randn(M, K, generator=g) / math.sqrt(K)).half()
    b = (torch.randn(K, N, generator=g) / math.sqrt(K)).half()
    want = ok.gemm(a, b)
    ad = a.t().contiguous().cuda().t() if ta else a.cuda()
    bd = b.t().contiguous().cuda().t() if tb else b.cuda()
    got = ops.matmul(ad, bd).cpu()
    assert _rel_err(got, want) <= 1e-2
    assert (got.float() - want.float()).abs().max().item() <= 1e-2


def test_gemm_bf16_many_tiles(ops):
    print("gemm bf16 many tiles", flush=True)
    g = _gen(19)
    a = (torch.randn(3072, 128, generator=g) / math.sqrt(128)).bfloat16()
    b = (torch.randn(128, 3328, generator=g) / math.sqrt(128)).bfloat16()
    got = ops.matmul(a.cuda(), b.cuda()).cpu()
    assert _rel_err(got, ok.gemm(a, b)) <= 1e-2


def test_grouped_gemm_reference_test_shapes(ops):
    """The reference's own grouped test: 1024, 512, 256 and 128 cubed (grouped_gemm.py:316-350)."""
    print("grouped gemm 1024/512/256/128 cubed", flush=True)
    g = _gen(16)
    A = [torch.rand(n, n, generator=g).half() for n in (1024, 512, 256, 128)]
    B = [torch.rand(n, n, generator=g).half() for n in (1024, 512, 256, 128)]
    want = ok.grouped_gemm(A, B)
    got = ops.lego_group_gemm_fn([a.cuda() for a in A], [b.cuda() for b in B])
    for c, w in zip(got, want):
        assert _rel_err(c.cpu(), w) <= 1e-2


def test_grouped_gemm_many_tiles_unsorted_depths(ops):
    """The headline grouped problem set at a sixteenth of its depth, in shuffled order: enough
    256 x 256 tiles for the one-workgroup-per-CU kernel, and the entry point's reordering by depth
    must hand every result back to its own problem."""
    print("grouped gemm many tiles, depths unsorted", flush=True)
    g = _gen(21)
    shapes = [(1024, 1024, 64), (4096, 1024, 128), (2048, 4096, 64), (4096, 4096, 64), (1024, 4096, 128),
              (2048, 2048, 64), (1024, 1024, 64), (4096, 2048, 64)]
    A = [(torch.randn(m, k, generator=g) / math.sqrt(k)).half() for m, n, k in shapes]
    B = [(torch.randn(k, n, generator=g) / math.sqrt(k)).half() for m, n, k in shapes]
    want = ok.grouped_gemm(A, B)
    got = ops.lego_group_gemm_fn([a.cuda() for a in A], [b.cuda() for b in B])
    for c, w in zip(got, want):
        assert c.shape == w.shape
        assert _rel_err(c.cpu(), w) <= 1e-2


# ---- GEMM shapes outside the tiled kernels: any M, N, K and alignment (matmul_sympy.py:69-70, 196-203) ----

@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.float8_e5m2, torch.float8_e4m3fn])
@pytest.mark.parametrize("M,N,K", [(1001, 263, 100), (1, 1, 1), (65, 64, 33), (1024, 512, 200), (1000, 264, 72),
                                   (1001, 264, 200), (1008, 528, 208), (300, 4104, 8), (2056, 2056, 1000)])
def test_gemm_any_shape_all_layouts(ops, dtype, M, N, K):
    """M, N, K of any size, the four operand layouts, with and without the fused leaky_relu.  Shapes whose
    operand rows are whole 16-byte chunks take the tiled kernels with ragged tiles and a masked last
    k-tile ((1024, 512, 200), (1000, 264, 72), (1008, 528, 208) for every element type, (1001, 264, 200)
    where A is stored row-major, K = 8 is a single, mostly masked k-tile); the others the kernel that
    moves one element per access."""
    print(f"gemm any shape {dtype} {M}x{N}x{K}", flush=True)
    g = _gen(41)
    a = (torch.randn(M, K, generator=g) / math.sqrt(K)).half().to(dtype)
    b = (torch.randn(K, N, generator=g) / math.sqrt(K)).half().to(dtype)
    want = a.float() @ b.float()
    tol = 2.0 ** -10           # the fp16 store's rounding + accumulation order
    for ta in (False, True):
        for tb in (False, True):
            ad = a.t().contiguous().cuda().t() if ta else a.cuda()
            bd = b.t().contiguous().cuda().t() if tb else b.cuda()
            got = ops.matmul(ad, bd)
            assert got.dtype == torch.float16 and got.shape == (M, N)      # the reference stores fp16 whatever the operands
            assert ((got.cpu().float() - want).abs() <= tol * want.abs() + 1e-3).all(), (ta, tb)
            if dtype == torch.bfloat16:
                own = ops.matmul(ad, bd, out_dtype=torch.bfloat16)
                assert own.dtype == torch.bfloat16
                assert ((own.cpu().float() - want).abs() <= 2.0 ** -8 * want.abs() + 1e-3).all(), (ta, tb)
            act = ops.matmul(ad, bd, activation="leaky_relu").cpu().float()
            want_act = torch.where(want >= 0, want, 0.01 * want)
            assert ((act - want_act).abs() <= tol * want_act.abs() + 1e-3).all(), (ta, tb)


def test_gemm_any_shape_is_exact_on_small_integers(ops):
    """Integer operands with exactly representable sums: every element of every ragged tile, bit for bit."""
    print("gemm any shape, integers", flush=True)
    g = _gen(42)
    M, N, K = 193, 131, 77
    a = torch.randint(-3, 4, (M, K), generator=g).half()
    b = torch.randint(-3, 4, (K, N), generator=g).half()
    want = (a.double() @ b.double()).half()
    for ta in (False, True):
        for tb in (False, True):
            ad = a.t().contiguous().cuda().t() if ta else a.cuda()
            bd = b.t().contiguous().cuda().t() if tb else b.cuda()
            assert torch.equal(ops.matmul(ad, bd).cpu(), want), (ta, tb)


def test_gemm_operands_at_any_element_alignment(ops):
    """Whole-tile shapes whose bases are not 16-byte aligned (views that start one element into a buffer)."""
    print("gemm misaligned bases", flush=True)
    g = _gen(43)
    M, N, K = 256, 256, 128
    a = (torch.randn(M * K + 1, generator=g) / math.sqrt(K)).half().cuda()[1:].view(M, K)
    b = (torch.randn(K * N + 3, generator=g) / math.sqrt(K)).half().cuda()[3:].view(K, N)
    assert a.data_ptr() % 16 and b.data_ptr() % 16
    got = ops.matmul(a, b).cpu()
    assert _rel_err(got, ok.gemm(a.cpu(), b.cpu())) <= 1e-2


def test_grouped_gemm_with_odd_problems(ops):
    """A grouped call with problems outside the tiled kernels falls back to one launch per problem."""
    print("grouped gemm, odd problems", flush=True)
    g = _gen(44)
    shapes = [(512, 256, 128), (1001, 263, 100), (64, 72, 200), (7, 5, 3)]
    A = [(torch.randn(m, k, generator=g) / math.sqrt(k)).half() for m, n, k in shapes]
    B = [(torch.randn(k, n, generator=g) / math.sqrt(k)).half() for m, n, k in shapes]
    want = ok.grouped_gemm(A, B)
    got = ops.lego_group_gemm_fn([a.cuda() for a in A], [b.cuda() for b in B])
    for c, w in zip(got, want):
        assert c.shape == w.shape
        assert ((c.cpu().float() - w.float()).abs() <= 2.0 ** -9 * w.float().abs() + 1e-3).all()


def test_grouped_gemm_entry_point_with_odd_problems(ops):
    """The C entry point itself (the wrapper sends odd problems elsewhere): a call with problems outside the tiled
    kernels falls back to one launch per problem, small integers bit for bit."""
    import ctypes
    from lego_amd import runtime
    print("grouped gemm entry point, odd problems", flush=True)
    g = _gen(46)
    shapes = [(256, 128, 64), (101, 63, 50), (64, 72, 200), (7, 5, 3)]
    A = [torch.randint(-2, 3, (m, k), generator=g).half().cuda() for m, n, k in shapes]
    B = [torch.randint(-2, 3, (k, n), generator=g).half().cuda() for m, n, k in shapes]
    C = [torch.empty(m, n, dtype=torch.half, device="cuda") for m, n, k in shapes]
    arr = ctypes.c_void_p * len(shapes)
    sz = (ctypes.c_int * (3 * len(shapes)))(*[v for s3 in shapes for v in s3])
    runtime.call("lego_hip_grouped_gemm_f16", arr(*[t.data_ptr() for t in A]), arr(*[t.data_ptr() for t in B]),
                 arr(*[t.data_ptr() for t in C]), sz, len(shapes), None)
    torch.cuda.synchronize()
    for a, b, c in zip(A, B, C):
        assert torch.equal(c.float(), a.float() @ b.float())


@pytest.mark.parametrize("count", [64, 65, 130])
def test_grouped_gemm_takes_any_number_of_problems(ops, count):
    """One launch carries 64 problems (the kernels' argument block); a call with more is enqueued as runs of 64 in
    order of decreasing depth, as the reference's host function takes any group size (grouped_gemm.py:120-162).
    All problems of different shape, many of a single ragged tile, depths unsorted; results come back in the
    caller's order."""
    print(f"grouped gemm, {count} problems", flush=True)
    g = _gen(45)
    shapes = [(8 * (1 + (5 * i) % 37), 8 * (1 + (7 * i) % 29), 8 * (1 + (3 * i) % 23)) for i in range(count)]
    A = [torch.randint(-2, 3, (m, k), generator=g).half() for m, n, k in shapes]
    B = [torch.randint(-2, 3, (k, n), generator=g).half() for m, n, k in shapes]
    got = ops.lego_group_gemm_fn([a.cuda() for a in A], [b.cuda() for b in B])
    for (m, n, k), a, b, c in zip(shapes, A, B, got):
        assert c.shape == (m, n)
        assert torch.equal(c.cpu().float(), a.float() @ b.float())      # small integers: exact
        assert torch.equal(c.cpu(), ok.gemm(a, b))


def test_grouped_gemm_of_130_problems_against_the_oracle(ops):
    """More than two runs' worth of problems with fractional data, each against the CPU oracle to the
    contract's relative error."""
    print("grouped gemm, 130 problems, random data", flush=True)
    g = _gen(46)
    shapes = [(64 * (1 + i % 5), 8 * (3 + (11 * i) % 40), 64 * (1 + (7 * i) % 9)) for i in range(130)]
    A = [(torch.randn(m, k, generator=g) / math.sqrt(k)).half() for m, n, k in shapes]
    B = [(torch.randn(k, n, generator=g) / math.sqrt(k)).half() for m, n, k in shapes]
    got = ops.lego_group_gemm_fn([a.cuda() for a in A], [b.cuda() for b in B])
    for a, b, c in zip(A, B, got):
        assert _rel_err(c.cpu(), ok.gemm(a, b)) <= 1e-2


def _grouped_call(entry, A, B, *extra):
    """Call a grouped entry point through the C ABI on device tensors; returns the results."""
    import ctypes
    from lego_amd import runtime
    C = [torch.empty(a.shape[0], b.shape[1], dtype=torch.half, device="cuda") for a, b in zip(A, B)]
    n = len(A)
    arr = ctypes.c_void_p * n
    sz = (ctypes.c_int * (3 * n))(*[v for a, b in zip(A, B) for v in (a.shape[0], b.shape[1], a.shape[1])])
    runtime.call(entry, arr(*[t.data_ptr() for t in A]), arr(*[t.data_ptr() for t in B]),
                 arr(*[t.data_ptr() for t in C]), sz, n, *extra,
                 ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
    torch.cuda.synchronize()
    return C


def test_grouped_gemm_headline_problem_set_at_full_depth(ops):
    """Config 5 as the benchmark builds it (seed 5: 8 problems from {1024, 2048, 4096}^3), whole: the
    launch splits its last tiles into halves.  Row panels of every problem against the CPU oracle
    (the first rows, rows 96..159 that straddle the two halves of a tile, the last rows), and the
    whole result against an fp32 product on the device."""
    print("grouped gemm config 5 at full depth", flush=True)
    g = _gen(5)
    idx = torch.randint(0, 3, (8, 3), generator=g)
    dims = [[(1024, 2048, 4096)[int(v)] for v in row] for row in idx]
    A = [(torch.randn(m, k, generator=g) / math.sqrt(k)).half() for m, n, k in dims]
    B = [(torch.randn(k, n, generator=g) / math.sqrt(k)).half() for m, n, k in dims]
    got = ops.lego_group_gemm_fn([a.cuda() for a in A], [b.cuda() for b in B])
    for (m, n, k), a, b, c in zip(dims, A, B, got):
        assert c.shape == (m, n)
        for r0 in (0, 96, m - 64):
            want = ok.gemm(a[r0:r0 + 64], b)
            assert _rel_err(c[r0:r0 + 64].cpu(), want) <= 1e-2, (m, n, k, r0)
            assert (c[r0:r0 + 64].cpu().float() - want.float()).abs().max().item() <= 1e-2
        ref = a.cuda().float() @ b.cuda().float()
        assert ((c.float() - ref).norm() / ref.norm()).item() <= 1e-2


def test_measurement_build_of_the_gemm_kernels_matches_and_stamps_in_order(ops):
    """The measurement build (time stamps at seven points of every tile) computes what the launched kernels
    compute, bit for bit, plain and grouped with halves, and every workgroup's stamps are in order."""
    print("gemm measurement build", flush=True)
    import ctypes
    import numpy as np
    from lego_amd import runtime
    g = _gen(53)
    shapes = [(4096, 4096, 128), (4096, 4096, 128), (2048, 4096, 64)]       # 256 + 256 + 128 tiles of 256 x 256: 2.5 rounds
    A = [(torch.randn(m, k, generator=g) / math.sqrt(k)).half().cuda() for m, n, k in shapes]
    B = [(torch.randn(k, n, generator=g) / math.sqrt(k)).half().cuda() for m, n, k in shapes]
    want = _grouped_call("lego_hip_grouped_gemm_f16", A, B)
    got = _grouped_call("lego_hip_grouped_gemm_f16_stamps", A, B)
    for c, w in zip(got, want):
        assert torch.equal(c, w)
    plan = (ctypes.c_int * 3)()
    sz = (ctypes.c_int * 9)(*[v for s in shapes for v in s])
    runtime.call("lego_hip_grouped_gemm_f16_plan", sz, 3, plan)
    assert plan[0] == 256
    wgs = plan[1] + plan[2]
    rows = np.zeros(8 * wgs, dtype=np.uint64)
    runtime.call("lego_hip_gemm_stamps_read", rows.ctypes.data_as(ctypes.c_void_p), wgs)
    st = rows.reshape(wgs, 8)[:, :7].astype(np.int64)
    assert (st[:, 0] > 0).all() and (np.diff(st, axis=1) >= 0).all()
    a, b = A[0][:1024], B[0][:, :768].contiguous()
    c0 = torch.empty(1024, 768, dtype=torch.half, device="cuda")
    c3 = torch.empty_like(c0)
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    for variant, c in ((0, c0), (3, c3)):
        runtime.call("lego_hip_gemm_f16_variant", ctypes.c_void_p(a.data_ptr()), ctypes.c_void_p(b.data_ptr()),
                     ctypes.c_void_p(c.data_ptr()), 1024, 768, 128, variant, stream)
    torch.cuda.synchronize()
    assert torch.equal(c0, c3)
    with pytest.raises(runtime.LegoHipError):
        runtime.call("lego_hip_gemm_stamps_read", rows.ctypes.data_as(ctypes.c_void_p), 8193)


@pytest.mark.parametrize("split", [0, 1, 7, 24, -1])
def test_grouped_gemm_split_tail_on_ragged_shapes(ops, split):
    """The launch with its last `split` tiles as two halves each, forced through the tuning entry
    point, on problems whose tiles are ragged: a last tile row of 8 rows (its lower half is empty), one
    of 136 rows (a lower half of 8 rows), ragged columns.  24 = every tile split; -1 = 128 x 128 tiles."""
    print(f"grouped gemm split tail {split}", flush=True)
    g = _gen(31)
    shapes = [(1000, 776, 192), (520, 264, 128), (136, 512, 64)]       # 16 + 6 + 2 tiles of 256 x 256
    A = [(torch.randn(m, k, generator=g) / math.sqrt(k)).half() for m, n, k in shapes]
    B = [(torch.randn(k, n, generator=g) / math.sqrt(k)).half() for m, n, k in shapes]
    want = ok.grouped_gemm(A, B)
    got = _grouped_call("lego_hip_grouped_gemm_f16_split", [a.cuda() for a in A], [b.cuda() for b in B], split)
    for c, w in zip(got, want):
        assert _rel_err(c.cpu(), w) <= 1e-2
        assert (c.cpu().float() - w.float()).abs().max().item() <= 1e-2


def test_grouped_gemm_split_matches_whole_tiles_bit_for_bit(ops):
    """A half-tile accumulates the same k-steps in the same order as the whole tile: same bits."""
    print("grouped gemm split vs whole", flush=True)
    g = _gen(32)
    shapes = [(2048, 1024, 512), (1024, 2048, 256), (512, 512, 128)]
    A = [(torch.randn(m, k, generator=g) / math.sqrt(k)).half().cuda() for m, n, k in shapes]
    B = [(torch.randn(k, n, generator=g) / math.sqrt(k)).half().cuda() for m, n, k in shapes]
    whole = _grouped_call("lego_hip_grouped_gemm_f16_split", A, B, 0)
    for split in (5, 68):
        for c, w in zip(_grouped_call("lego_hip_grouped_gemm_f16_split", A, B, split), whole):
            assert torch.equal(c, w)


@pytest.mark.parametrize("split", [0, 40, 300])
def test_grouped_gemm_launch_order_over_depth_classes(ops, split):
    """Workgroup ids are dealt to tiles per class of equal depth, in rounds of 256 with a contiguous run per
    XCD: a class that starts at a flat index that is not a multiple of 8 (3 tiles come before it), one of
    289 + 20 tiles (a whole round, then a remainder of 53 that is not a multiple of 8), one of 72 + 24 (a
    remainder that is), and the same with the last tiles as halves, so that the whole tiles of a class stop
    and its halves start in the middle of it.  Every tile must be computed exactly once: against the oracle."""
    print(f"grouped gemm launch order over depth classes, split {split}", flush=True)
    g = _gen(61)
    shapes = [(768, 256, 192), (4352, 4352, 128), (1024, 1280, 128), (2048, 2304, 64), (1536, 1024, 64)]
    A = [(torch.randn(m, k, generator=g) / math.sqrt(k)).half() for m, n, k in shapes]
    B = [(torch.randn(k, n, generator=g) / math.sqrt(k)).half() for m, n, k in shapes]
    want = ok.grouped_gemm(A, B)
    got = _grouped_call("lego_hip_grouped_gemm_f16_split", [a.cuda() for a in A], [b.cuda() for b in B], split)
    for c, w in zip(got, want):
        assert _rel_err(c.cpu(), w) <= 1e-2
        assert (c.cpu().float() - w.float()).abs().max().item() <= 1e-2


def test_gemm_headline_shape_8192_cubed(ops):
    """Config 4 at full size: 1024 tiles, 128 k-steps each, operands 128 MiB apart as two consecutive
    allocations are.  Two 256-row panels (the first tile row and one in the middle of the launch order's
    last group) against the CPU oracle."""
    print("gemm 8192 cubed", flush=True)
    n = 8192
    g = _gen(4)
    a = (torch.randn(n, n, generator=g) / math.sqrt(n)).half()
    b = (torch.randn(n, n, generator=g) / math.sqrt(n)).half()
    c = ops.matmul(a.cuda(), b.cuda())
    for r0 in (0, 7424):
        want = ok.gemm(a[r0:r0 + 256], b)
        got = c[r0:r0 + 256].cpu()
        assert _rel_err(got, want) <= 1e-2
        assert (got.float() - want.float()).abs().max().item() <= 1e-2


def test_kernels_run_on_the_callers_stream(ops):
    """The wrappers enqueue on torch's current stream: work issued on a side stream is ordered after that
    stream's earlier work (the input is produced there) and is complete once the stream is."""
    print("side stream", flush=True)
    side = torch.cuda.Stream()          # default priority
    g = _gen(25)
    x_host = (2.0 * torch.randn(512, 4096, generator=g)).half()
    a_host = (torch.randn(512, 256, generator=g) / 16).half()
    b_host = (torch.randn(256, 512, generator=g) / 16).half()
    with torch.cuda.stream(side):
        x = x_host.cuda(non_blocking=True) * 1.0          # produced on the side stream
        y = ops.softmax(x)
        t = ops.transpose(y)
        c = ops.matmul(a_host.cuda(non_blocking=True), b_host.cuda(non_blocking=True))
    side.synchronize()
    want = ok.softmax(x_host)
    assert (y.cpu().float() - want.float()).abs().max().item() <= TOL
    assert torch.equal(t.cpu(), y.cpu().t().contiguous())
    assert _rel_err(c.cpu(), ok.gemm(a_host, b_host)) <= 1e-2


def test_entry_points_replay_from_a_hip_graph(ops):
    """Nothing behind the C ABI allocates, synchronises or keeps state, so a chain of calls can be
    captured once and replayed: every replay, on new input, matches the eager result."""
    print("graph capture and replay", flush=True)
    g = _gen(26)
    M, N = 256, 2048
    x = torch.zeros(M, N, dtype=torch.half, device="cuda")
    w = (1 + 0.1 * torch.randn(N, generator=g)).half().cuda()
    b = (0.1 * torch.randn(N, generator=g)).half().cuda()
    wm = (torch.randn(N, 512, generator=g) / math.sqrt(N)).half().cuda()

    def chain(inp):
        y, _, _ = ops.layer_norm_fwd(inp, w, b, 1e-5)
        z = ops.matmul(y, wm)
        return ops.transpose(ops.softmax(z))

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        chain(x)                         # warm-up outside the capture
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        out = chain(x)
    for trial in range(3):
        fresh = (2.0 * torch.randn(M, N, generator=g)).half().cuda()
        x.copy_(fresh)
        graph.replay()
        torch.cuda.synchronize()
        got = out.clone()
        want = chain(fresh)              # eager work between the replays
        torch.cuda.synchronize()
        assert torch.equal(got, want), trial


def test_gemm_offsets_beyond_32_bits(ops):
    """Operands and results of more than 2^32 elements: tile offsets are 64-bit.  The last row tile,
    whose offset in A (first case) or in C (second case) does not fit 32 bits, is checked against the oracle."""
    print("gemm with more than 2^32 elements per matrix", flush=True)
    g = torch.Generator(device="cuda").manual_seed(27)
    M, K, N = 65536 + 256, 65536, 256
    a = torch.empty(M, K, device="cuda", dtype=torch.half).normal_(0, 1 / 256, generator=g)
    b = torch.empty(K, N, device="cuda", dtype=torch.half).normal_(0, 1 / 256, generator=g)
    c = ops.matmul(a, b)
    for rows in (slice(0, 256), slice(M - 256, M)):
        assert _rel_err(c[rows].cpu(), ok.gemm(a[rows].cpu(), b.cpu())) <= 1e-2
    del a, b, c
    M, K, N = 65536 + 256, 64, 65536
    a = torch.empty(M, K, device="cuda", dtype=torch.half).normal_(0, 1 / 8, generator=g)
    b = torch.empty(K, N, device="cuda", dtype=torch.half).normal_(0, 1 / 8, generator=g)
    c = ops.matmul(a, b)
    for rows in (slice(0, 256), slice(M - 256, M)):
        assert _rel_err(c[rows].cpu(), ok.gemm(a[rows].cpu(), b.cpu())) <= 1e-2


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("M,N,K", [(16, 2048, 2048), (1, 1024, 4096), (100, 264, 3000), (256, 256, 16384), (24, 4096, 2056),
                                   (2048, 16, 2048), (130, 130, 8200)])
def test_gemm_split_along_k(ops, dtype, M, N, K):
    """Products of few tiles get a workspace from the wrapper and are split along K: skinny operands, a long
    K, ragged tiles and a ragged last k-tile (which falls to the last part).  Small integers (thinned out
    so that every sum stays exact in 16 bits) in all four layouts, with and without the fused
    activation; then random operands against the CPU oracle."""
    import ctypes
    from lego_amd import runtime
    print(f"gemm split along k {dtype} {M}x{N}x{K}", flush=True)
    need = ctypes.c_ulonglong(0)
    runtime.call("lego_hip_gemm_workspace_bytes", M, N, K, ctypes.byref(need))
    assert need.value > 0 and (N % 8 or K % 8 or need.value % (128 * 128 * 4) == 0)
    g = _gen(81)
    a = torch.randint(-2, 3, (M, K), generator=g).float()
    b = torch.randint(-2, 3, (K, N), generator=g).float()
    a = a * (torch.rand(M, K, generator=g) < min(1.0, 500.0 / K))      # about 500 non-zero terms of -4..4 per sum
    want = a @ b
    assert want.abs().max().item() <= 256          # exact in bfloat16 too
    for ta in (False, True):
        for tb in (False, True):
            if ta and M % 8:
                continue                # a transposed A of such an M is outside the tiled kernels
            ad = a.to(dtype).cuda()
            bd = b.to(dtype).cuda()
            ad = ad.t().contiguous().t() if ta else ad
            bd = bd.t().contiguous().t() if tb else bd
            assert torch.equal(ops.matmul(ad, bd).cpu().float(), want), (ta, tb)
            leaky = torch.where(want >= 0, want, 0.01 * want).half().float()
            assert torch.equal(ops.matmul(ad, bd, activation="leaky_relu").cpu().float(), leaky), (ta, tb)
    a = (torch.randn(M, K, generator=g) / math.sqrt(K)).to(dtype)
    b = (torch.randn(K, N, generator=g) / math.sqrt(K)).to(dtype)
    got = ops.matmul(a.cuda(), b.cuda()).cpu()
    assert _rel_err(got, ok.gemm(a, b)) <= 1e-2


def test_gemm_split_along_k_entry_point(ops):
    """lego_hip_gemm_ex_ws through the C ABI: with the workspace it asks for it is bit-identical from call to
    call (the parts are added in a fixed order) and within rounding of the plain entry point; with none, or a
    short one, it IS the plain entry point; shapes with enough tiles ask for no workspace."""
    import ctypes
    from lego_amd import runtime
    print("gemm split along k, entry point", flush=True)
    M, N, K = 64, 1024, 8192
    g = _gen(82)
    a = (torch.randn(M, K, generator=g) / math.sqrt(K)).half().cuda()
    b = (torch.randn(K, N, generator=g) / math.sqrt(K)).half().cuda()
    need = ctypes.c_ulonglong(0)
    runtime.call("lego_hip_gemm_workspace_bytes", M, N, K, ctypes.byref(need))
    assert need.value > 0
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    p = lambda t: ctypes.c_void_p(t.data_ptr())
    plain = torch.empty(M, N, dtype=torch.half, device="cuda")
    runtime.call("lego_hip_gemm_f16_ex", p(a), p(b), p(plain), M, N, K, 0, 0, 0, stream)
    ws = torch.empty(need.value // 4, dtype=torch.float32, device="cuda")
    outs = []
    for fill in (0.0, float("nan")):            # whatever the workspace held
        ws.fill_(fill)
        c = torch.empty(M, N, dtype=torch.half, device="cuda")
        runtime.call("lego_hip_gemm_ex_ws", 0, p(a), p(b), p(c), M, N, K, 0, 0, 0, p(ws), need, stream)
        outs.append(c)
    assert torch.equal(outs[0], outs[1])
    assert (outs[0].float() - plain.float()).abs().max().item() <= 2e-3      # another summation order, one rounding
    for workspace, size in ((None, 0), (p(ws), need.value - 1)):
        c = torch.empty(M, N, dtype=torch.half, device="cuda")
        runtime.call("lego_hip_gemm_ex_ws", 0, p(a), p(b), p(c), M, N, K, 0, 0, 0, workspace, ctypes.c_ulonglong(size), stream)
        assert torch.equal(c, plain)
    for shape in ((4096, 4096, 4096), (2048, 1024, 64), (128, 128, 256)):
        runtime.call("lego_hip_gemm_workspace_bytes", *shape, ctypes.byref(need))
        assert need.value == 0, shape
    with pytest.raises(runtime.LegoHipError):
        runtime.call("lego_hip_gemm_ex_ws", 2, p(a), p(b), p(plain), M, N, K, 0, 0, 0, p(ws), need, stream)   # 8-bit: no


@pytest.mark.parametrize("element,dtype", [(0, torch.float16), (1, torch.bfloat16), (4, torch.bfloat16)])
@pytest.mark.parametrize("M,N,K", [(193, 131, 77), (257, 264, 1001), (1001, 263, 104), (5, 7, 3), (520, 1027, 2049)])
def test_gemm_on_zero_padded_copies(ops, element, dtype, M, N, K):
    """lego_hip_gemm_ex_ws through the C ABI for N or K that is not a multiple of 8: the tiled kernels run on
    zero-padded copies in the workspace.  Small integers, so every layout gives the exact product whatever the
    workspace held; nothing outside C and the workspace is written; the answer is that of the plain entry point;
    operands may start at any element."""
    import ctypes
    from lego_amd import runtime
    print(f"gemm on padded copies {dtype} element {element} {M}x{N}x{K}", flush=True)
    g = _gen(83)
    a = torch.randint(-2, 3, (M, K), generator=g).to(dtype)
    b = torch.randint(-2, 3, (K, N), generator=g).to(dtype)
    if K > 1000:       # keep the sums exact in the result type
        a = a * (torch.rand(M, K, generator=g) < 200.0 / K).to(dtype)
    want = (a.double() @ b.double())
    out_dtype = torch.bfloat16 if element == 1 else torch.float16
    assert want.abs().max().item() <= 256
    need = ctypes.c_ulonglong(0)
    runtime.call("lego_hip_gemm_workspace_bytes", M, N, K, ctypes.byref(need))
    assert need.value >= 2 * (M * K + K * N + M * N)
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    p = lambda t: ctypes.c_void_p(t.data_ptr())
    ws = torch.empty(need.value // 4 + 64, dtype=torch.float32, device="cuda")
    for ta in (0, 1):
        for tb in (0, 1):
            for shift in (0, 3):          # operands and result 16-byte aligned, or three elements past it
                def place(t):
                    buf = torch.zeros(t.numel() + 8, dtype=t.dtype, device="cuda")
                    buf[shift:shift + t.numel()] = t.reshape(-1).cuda()
                    return buf[shift:shift + t.numel()]
                ad = place(a.t().contiguous() if ta else a)
                bd = place(b.t().contiguous() if tb else b)
                ws.fill_(float("nan"))
                cbuf = torch.full((M * N + 2048,), 7.0, dtype=out_dtype, device="cuda")
                c = cbuf[1024 + shift:1024 + shift + M * N]
                runtime.call("lego_hip_gemm_ex_ws", element, p(ad), p(bd), p(c), M, N, K, ta, tb, 0, p(ws), need, stream)
                torch.cuda.synchronize()
                assert torch.equal(c.view(M, N).cpu().double(), want), (ta, tb, shift)
                assert (cbuf[:1024 + shift] == 7.0).all() and (cbuf[1024 + shift + M * N:] == 7.0).all()
                assert torch.isnan(ws[need.value // 4:]).all()          # nothing past the bytes it asked for
    # no workspace: the plain entry point's answer
    ad, bd = a.cuda(), b.cuda()
    c = torch.empty(M, N, dtype=out_dtype, device="cuda")
    runtime.call("lego_hip_gemm_ex_ws", element, p(ad), p(bd), p(c), M, N, K, 0, 0, 0, None, ctypes.c_ulonglong(0), stream)
    assert torch.equal(c.cpu().double(), want)


def test_gemm_rejects_bad_arguments(ops):
    with pytest.raises(ValueError):          # inner dimensions differ
        ops.matmul(torch.zeros(100, 64, device="cuda", dtype=torch.half),
                   torch.zeros(72, 256, device="cuda", dtype=torch.half))
    with pytest.raises(ValueError):          # neither the operand nor its transpose is contiguous
        ops.matmul(torch.zeros(100, 128, device="cuda", dtype=torch.half)[:, ::2],
                   torch.zeros(64, 256, device="cuda", dtype=torch.half))
    with pytest.raises(NotImplementedError):
        ops.matmul(torch.zeros(256, 64, device="cuda", dtype=torch.half),
                   torch.zeros(64, 256, device="cuda", dtype=torch.half), activation="gelu")


@pytest.mark.parametrize("ta,tb", [(False, True), (True, False), (True, True)])
@pytest.mark.parametrize("M,N,K", [(256, 256, 64), (512, 768, 320), (1024, 256, 1024)])
def test_gemm_transposed_operands(ops, ta, tb, M, N, K):
    """The reference's TA/TB variants: operands are .T views of contiguous tensors."""
    print(f"gemm ta={ta} tb={tb} {M}x{N}x{K}", flush=True)
    g = _gen(9)
    a = (torch.randn(M, K, generator=g) / math.sqrt(K)).half()
    b = (torch.randn(K, N, generator=g) / math.sqrt(K)).half()
    want = ok.gemm(a, b)
    ad = a.t().contiguous().cuda().t() if ta else a.cuda()
    bd = b.t().contiguous().cuda().t() if tb else b.cuda()
    assert ad.shape == (M, K) and bd.shape == (K, N)
    got = ops.matmul(ad, bd).cpu()
    assert _rel_err(got, want) <= 1e-2
    assert (got.float() - want.float()).abs().max().item() <= 1e-2


def test_gemm_transposed_integer_exact(ops):
    g = _gen(10)
    a = torch.randint(-2, 3, (512, 256), generator=g).half()
    b = torch.randint(-2, 3, (256, 768), generator=g).half()
    want = a.double() @ b.double()
    for ta in (False, True):
        for tb in (False, True):
            print(f"gemm integer exact ta={ta} tb={tb}", flush=True)
            ad = a.t().contiguous().cuda().t() if ta else a.cuda()
            bd = b.t().contiguous().cuda().t() if tb else b.cuda()
            assert torch.equal(ops.matmul(ad, bd).cpu().double(), want)


@pytest.mark.parametrize("ta,tb", [(False, False), (False, True), (True, False), (True, True)])
def test_gemm_bf16_matches_oracle(ops, ta, tb):
    """bfloat16 operands and result: rel-err <= 1e-2 against fp32 accumulation (bf16 has 8
    significand bits, so the rounding of the result alone is up to 2^-9 relative)."""
    M, N, K = 512, 768, 320
    print(f"gemm bf16 ta={ta} tb={tb} {M}x{N}x{K}", flush=True)
    g = _gen(11)
    a = (torch.randn(M, K, generator=g) / math.sqrt(K)).bfloat16()
    b = (torch.randn(K, N, generator=g) / math.sqrt(K)).bfloat16()
    want = ok.gemm(a, b)
    ad = a.t().contiguous().cuda().t() if ta else a.cuda()
    bd = b.t().contiguous().cuda().t() if tb else b.cuda()
    got = ops.matmul(ad, bd, out_dtype=torch.bfloat16)
    assert got.dtype == torch.bfloat16
    assert _rel_err(got.cpu(), want) <= 1e-2
    # round-to-nearest-even of the fp32 accumulator: at most one bf16 spacing from the oracle
    assert (got.cpu().float() - want.float()).abs().max().item() <= 2.0 ** -7
    # the default is the reference's: an fp16 result whatever the operands' 16-bit type (matmul_sympy.py:136)
    half = ops.matmul(ad, bd)
    assert half.dtype == torch.float16
    exact = a.float() @ b.float()
    assert ((half.cpu().float() - exact).abs() <= 2.0 ** -10 * exact.abs() + 1e-4).all()


def test_gemm_bf16_integer_exact(ops):
    """Operands in {-1, 0, 1} and K = 256: every sum is an integer of magnitude <= 256, exact in
    fp32 and in bf16."""
    print("gemm bf16 integer exact", flush=True)
    g = _gen(12)
    a = torch.randint(-1, 2, (512, 256), generator=g).bfloat16()
    b = torch.randint(-1, 2, (256, 768), generator=g).bfloat16()
    want = a.double() @ b.double()
    for ta in (False, True):
        for tb in (False, True):
            ad = a.t().contiguous().cuda().t() if ta else a.cuda()
            bd = b.t().contiguous().cuda().t() if tb else b.cuda()
            assert torch.equal(ops.matmul(ad, bd).cpu().double(), want)


@pytest.mark.parametrize("fp8", [torch.float8_e5m2, torch.float8_e4m3fn])
@pytest.mark.parametrize("ta,tb", [(False, False), (False, True), (True, False), (True, True)])
def test_gemm_fp8_matches_oracle(ops, fp8, ta, tb):
    """8-bit operands (the reference casts randn fp16 tensors to float8_e5m2, matmul_sympy.py:346-364):
    products of two fp8 values are exact in fp32, so the result differs from the fp32 product of
    the same fp8 values only by accumulation order and the fp16 rounding of the result."""
    M, N, K = 512, 768, 384
    print(f"gemm {fp8} ta={ta} tb={tb} {M}x{N}x{K}", flush=True)
    g = _gen(13)
    a = torch.randn(M, K, generator=g).half().to(fp8)
    b = torch.randn(K, N, generator=g).half().to(fp8)
    want = (a.float() @ b.float())
    ad = a.t().contiguous().cuda().t() if ta else a.cuda()
    bd = b.t().contiguous().cuda().t() if tb else b.cuda()
    got = ops.matmul(ad, bd)
    assert got.dtype == torch.float16 and got.shape == (M, N)
    assert _rel_err(got.cpu(), want) <= 1e-2
    assert (got.cpu().float() - want).abs().max().item() <= 0.125     # the reference's own atol


def test_gemm_fp8_integer_exact(ops):
    """Operands in {-2..2} (exact in both 8-bit formats), K = 256: every sum is an integer below
    2048, exact in fp32 and fp16.  A lane/byte mix-up between the operands changes the integers."""
    g = _gen(14)
    a = torch.randint(-2, 3, (512, 256), generator=g).float()
    b = torch.randint(-2, 3, (256, 768), generator=g).float()
    want = a.double() @ b.double()
    for fp8 in (torch.float8_e5m2, torch.float8_e4m3fn):
        for ta in (False, True):
            for tb in (False, True):
                print(f"gemm {fp8} integer exact ta={ta} tb={tb}", flush=True)
                a8, b8 = a.to(fp8), b.to(fp8)
                ad = a8.t().contiguous().cuda().t() if ta else a8.cuda()
                bd = b8.t().contiguous().cuda().t() if tb else b8.cuda()
                assert torch.equal(ops.matmul(ad, bd).cpu().double(), want)


def test_gemm_leaky_relu_epilogue(ops):
    print("gemm leaky_relu", flush=True)
    g = _gen(8)
    a = (torch.randn(512, 256, generator=g) / 16).half()
    b = (torch.randn(256, 512, generator=g) / 16).half()
    want = torch.nn.functional.leaky_relu(a.float() @ b.float(), 0.01).half()
    got = ops.matmul(a.cuda(), b.cuda(), activation="leaky_relu").cpu()
    assert _rel_err(got, want) <= 1e-2
    assert (got.float() - want.float()).abs().max().item() <= 1e-2
    assert (got < 0).any() and (got > 0).any()


def test_tuner_compares_the_alternatives(ops, capsys):
    """`python -m lego_amd.tune`: every alternative behind a dispatch threshold through its tuning entry point."""
    print("tuner", flush=True)
    from lego_amd import tune
    assert tune.main(["transpose", "--dtype", "f32", "--shapes", "1000x1004"]) == 0
    assert tune.main(["rows", "--shapes", "512x1024"]) == 0
    assert tune.main(["gemm", "--shapes", "512x512x256"]) == 0
    out = capsys.readouterr().out
    assert "dispatch:" in out and "ragged" in out and "4 waves:" in out and "16x16x32, 4 waves:" in out
