"""3-D stencils on row-major and bricks storage: oracle pins on the CPU, parity on the GPU."""
import numpy as np
import pytest
import torch

from oracle import kernels as ok


def _coefficients(radius):
    """The reference program's coefficient cube (benchmarks/cuda/bricks/main_tmp.cu:139-150)."""
    c = np.zeros((8, 8, 8), dtype=np.float32)
    for a in range(7):
        for b in range(7):
            for d in range(7):
                c[a, b, d] = 1.0 / (1.0 + (a - radius) ** 2 + (b - radius) ** 2 + (d - radius) ** 2)
    c[radius, radius, radius] += 1.0
    return c


def test_oracle_f3d_matches_point_loops():
    rng = np.random.default_rng(1)
    for n, r in ((8, 1), (10, 2)):
        x = rng.uniform(-1, 1, (n, n, n)).astype(np.float32)
        c = rng.uniform(-1, 1, (8, 8, 8)).astype(np.float32)
        want = np.zeros((n, n, n))
        for p in np.ndindex(n, n, n):
            if all(r <= q < n - r for q in p):
                s = float(x[p]) * float(c[r, r, r])
                for d in np.ndindex(2 * r + 1, 2 * r + 1, 2 * r + 1):
                    s += float(x[p[0] + d[0] - r, p[1] + d[1] - r, p[2] + d[2] - r]) * float(c[d])
                want[p] = s
        assert np.allclose(ok.stencil_f3d(x, c, r), want, rtol=0, atol=1e-12)


def test_oracle_stencils_on_a_constant_field():
    """A constant field makes both stencils a sum of coefficients."""
    n = 16
    x = np.full((n, n, n), 2.0, dtype=np.float32)
    for r in (1, 2, 3):
        c = _coefficients(r)
        got = ok.stencil_f3d(x, c, r)
        window = c[:2 * r + 1, :2 * r + 1, :2 * r + 1].astype(np.float64).sum() + float(c[r, r, r])
        assert np.allclose(got[r:n - r, r:n - r, r:n - r], 2.0 * window)
        assert got[0].max() == 0 and got[:, :, n - 1].max() == 0
        cl = np.arange(1, r + 2, dtype=np.float32)
        gl = ok.stencil_laplacian(x, cl, r)
        assert np.allclose(gl[r:n - r, r:n - r, r:n - r], 2.0 * (cl[0] + 6 * cl[1:].sum()))


def test_oracle_laplacian_of_a_quadratic():
    """f = x^2 + 2 y^2 + 3 z^2 with c = (-6, 1): the 7-point Laplacian is exactly 2 + 4 + 6."""
    n = 12
    g = np.arange(n, dtype=np.float64)
    f = (g[:, None, None] ** 2 + 2 * g[None, :, None] ** 2 + 3 * g[None, None, :] ** 2).astype(np.float32)
    got = ok.stencil_laplacian(f, np.array([-6.0, 1.0], dtype=np.float32), 1)
    assert np.allclose(got[1:-1, 1:-1, 1:-1], 12.0)


def test_bricks_order_matches_the_reference_offsets():
    """benchmarks/cuda/bricks/main.cu:91 holds the offset of point (bx, by, bz, i, j, k) of the
    384^3 bricks layout: 1179648*bx + 24576*by + 512*bz + 64*i + 8*j + k."""
    n = 384
    order = ok.bricks_order(n)
    rng = np.random.default_rng(2)
    for _ in range(200):
        bx, by, bz = rng.integers(0, 48, 3)
        i, j, k = rng.integers(0, 8, 3)
        assert order[8 * bx + i, 8 * by + j, 8 * bz + k] == 1179648 * bx + 24576 * by + 512 * bz + 64 * i + 8 * j + k
    small = ok.bricks_order(16)
    assert sorted(small.ravel().tolist()) == list(range(16 ** 3))


def test_shell_rows_in_lds_spread_over_the_banks():
    """The sixteen lanes that a 16-byte LDS access serves together read rows (i, 0..7) and (i+1, 0..7) of the
    shell: with 20-word rows and the padded planes of the kernel they start in sixteen different groups of
    four banks, for every neighbour offset (radius 1 and 3; the radius-2 shell is left unpadded on purpose)."""
    from lego_amd.kernels import stencil
    words = stencil.ROW_WORDS
    for radius in (1, 3):
        h = 8 + 2 * radius
        plane = stencil.shell_plane(radius)
        assert plane % 4 == 0 and plane >= h * words
        for di in range(-radius, radius + 1):
            for dj in range(-radius, radius + 1):
                for first in range(0, 64, 16):
                    groups = set()
                    for lane in range(first, first + 16):
                        i, j = divmod(lane, 8)
                        word = plane * (i + radius + di) + words * (j + radius + dj)
                        assert word % 4 == 0
                        groups.add((word // 4) % 16)
                    assert len(groups) == 16
    # the star kernel's rows of eight words in planes of 8*H + 4 words
    for radius in (1, 2, 3):
        h = 8 + 2 * radius
        plane = 8 * h + 4
        for first in range(0, 64, 16):
            for di, dj in ((0, 0), (radius, 0), (-radius, 0), (0, radius), (0, -radius)):
                groups = {(plane * (lane // 8 + radius + di) + 8 * (lane % 8 + radius + dj)) // 4 % 16 for lane in range(first, first + 16)}
                assert len(groups) == 16


def _to_bricks(x, order):
    out = torch.empty(x.numel(), dtype=x.dtype)
    out[torch.from_numpy(order).reshape(-1)] = x.reshape(-1)
    return out.view(x.shape)


def _from_bricks(y, order):
    return y.reshape(-1)[torch.from_numpy(order).reshape(-1)].view(y.shape)


@pytest.mark.gpu
@pytest.mark.parametrize("bricks", [False, True])
@pytest.mark.parametrize("n,radius", [(8, 1), (8, 3), (16, 1), (24, 2), (64, 1), (64, 2), (32, 3), (128, 1)])
def test_gpu_f3d_matches_oracle(n, radius, bricks):
    from lego_amd import ops
    print(f"f3d n={n} radius={radius} bricks={bricks}", flush=True)
    g = torch.Generator().manual_seed(30 + n + radius)
    x = torch.rand(n, n, n, generator=g) * 2 - 1
    c = torch.from_numpy(_coefficients(radius))
    want = torch.from_numpy(ok.stencil_f3d(x.numpy(), c.numpy(), radius)).float()
    order = ok.bricks_order(n)
    xin = _to_bricks(x, order) if bricks else x
    got = ops.stencil_f3d(xin.cuda(), c.cuda(), radius, bricks).cpu()
    got = _from_bricks(got, order) if bricks else got
    assert (got - want).abs().max().item() <= 2e-5 * (2 * radius + 1) ** 3


@pytest.mark.gpu
@pytest.mark.parametrize("bricks", [False, True])
@pytest.mark.parametrize("n,radius", [(8, 1), (8, 3), (16, 1), (24, 3), (64, 2), (64, 3), (128, 1),
                                      (16, 4), (40, 4), (64, 4)])      # radius 4: the reference's largest (result/cuda/bricks-laplace.txt)
def test_gpu_laplacian_matches_oracle(n, radius, bricks):
    from lego_amd import ops
    print(f"laplacian n={n} radius={radius} bricks={bricks}", flush=True)
    g = torch.Generator().manual_seed(40 + n + radius)
    x = torch.rand(n, n, n, generator=g) * 2 - 1
    c = torch.tensor([-6.0, 1.0, 0.5, 0.25, 0.125])[:radius + 1].contiguous()
    want = torch.from_numpy(ok.stencil_laplacian(x.numpy(), c.numpy(), radius)).float()
    order = ok.bricks_order(n)
    xin = _to_bricks(x, order) if bricks else x
    got = ops.stencil_laplacian(xin.cuda(), c.cuda(), radius, bricks).cpu()
    got = _from_bricks(got, order) if bricks else got
    assert (got - want).abs().max().item() <= 1e-5


@pytest.mark.gpu
@pytest.mark.parametrize("kind,radius", [("f3d", 1), ("f3d", 3), ("laplacian", 1), ("laplacian", 3), ("laplacian", 4)])
def test_gpu_stencils_full_size_match_oracle_on_slabs(kind, radius):
    """The reference's size, 384^3, both storage orders, against the float64 oracle on three slabs of 16
    planes (the first, one across the middle of the brick grid, the last): the oracle of a slab widened
    by the radius equals the oracle of the cube on the slab's own planes."""
    from lego_amd import ops
    print(f"{kind} 384^3 radius {radius} against the oracle on slabs", flush=True)
    n = 384
    x = torch.rand(n, n, n, generator=torch.Generator().manual_seed(51 + radius)) * 2 - 1
    if kind == "f3d":
        c = torch.from_numpy(_coefficients(radius))
        call, oracle, tol = ops.stencil_f3d, ok.stencil_f3d, 2e-5 * (2 * radius + 1) ** 3
    else:
        c = torch.tensor([-6.0, 1.0, 0.5, 0.25, 0.125])[:radius + 1].contiguous()
        call, oracle, tol = ops.stencil_laplacian, ok.stencil_laplacian, 1e-5
    order = ok.bricks_order(n)
    rowmajor = call(x.cuda(), c.cuda(), radius, False).cpu()
    bricks = _from_bricks(call(_to_bricks(x, order).cuda(), c.cuda(), radius, True).cpu(), order)
    assert torch.equal(rowmajor, bricks)
    for lo, hi in ((0, 16), (184, 200), (n - 16, n)):
        a, b = max(0, lo - radius), min(n, hi + radius)
        want = torch.from_numpy(oracle(x[a:b].numpy(), c.numpy(), radius)).float()
        # planes of the slab that are boundary planes of the widened slab but not of the cube are not the cube's
        keep = slice(lo - a, hi - a)
        got = rowmajor[lo:hi]
        ref = want[keep]
        if lo == 0:
            assert got[:radius].abs().max().item() == 0          # the cube's own boundary planes are not written
            got, ref = got[radius:], ref[radius:]
        if hi == n:
            assert got[-radius:].abs().max().item() == 0
            got, ref = got[:-radius], ref[:-radius]
        assert (got - ref).abs().max().item() <= tol, (lo, hi)


@pytest.mark.gpu
def test_gpu_stencils_full_size_agree_between_layouts():
    """The reference's size, 384^3: both storage orders give the same field, bit for bit (the
    arithmetic of a point does not depend on where its neighbours are stored)."""
    from lego_amd import ops
    print("stencils 384^3, row-major vs bricks", flush=True)
    n = 384
    x = torch.rand(n, n, n, generator=torch.Generator().manual_seed(50)) * 2 - 1
    c = torch.from_numpy(_coefficients(1)).cuda()
    order = ok.bricks_order(n)
    a = ops.stencil_f3d(x.cuda(), c, 1, False).cpu()
    b = _from_bricks(ops.stencil_f3d(_to_bricks(x, order).cuda(), c, 1, True).cpu(), order)
    assert torch.equal(a, b)
    assert a[0].abs().max().item() == 0 and a[1:-1, 1:-1, 1:-1].abs().max().item() > 0


@pytest.mark.gpu
def test_gpu_stencil_rejects_bad_arguments():
    from lego_amd import ops
    from lego_amd.runtime import LegoHipError
    x = torch.zeros(16, 16, 16, device="cuda")
    c = torch.zeros(8, 8, 8, device="cuda")
    with pytest.raises(LegoHipError):
        ops.stencil_f3d(x, c, radius=4)
    with pytest.raises(LegoHipError):
        ops.stencil_f3d(torch.zeros(12, 12, 12, device="cuda"), c, radius=1)
    # an `out` the kernel could not write through is refused before the launch
    for bad in (torch.zeros(16, 16, 16), torch.zeros(16, 16, 16, device="cuda", dtype=torch.half),
                torch.zeros(8, 16, 16, device="cuda"), torch.zeros(16, 16, 32, device="cuda")[:, :, ::2], x):
        with pytest.raises(ValueError):
            ops.stencil_f3d(x, c, radius=1, out=bad)
        with pytest.raises(ValueError):
            ops.stencil_laplacian(x, torch.zeros(2, device="cuda"), radius=1, out=bad)
