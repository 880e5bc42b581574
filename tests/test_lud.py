"""LU decomposition without pivoting: oracle pins on the CPU, parity on the GPU."""
import numpy as np
import pytest
import scipy.linalg
import torch

from lego_amd.kernels import lud as lud_gen
from oracle import kernels as ok


def _dominant(n, seed):
    """Strictly column-diagonally-dominant: partial pivoting never swaps, so a library LU with
    pivoting is the decomposition without pivoting."""
    rng = np.random.default_rng(seed)
    a = rng.uniform(-1, 1, (n, n))
    a[np.arange(n), np.arange(n)] = np.abs(a).sum(axis=0) + 1.0
    return a


def test_oracle_matches_scipy_on_dominant_matrices():
    for n in (5, 64, 130):
        a = _dominant(n, n)
        p, l, u = scipy.linalg.lu(a)
        assert np.array_equal(p, np.eye(n))
        got = ok.lud(a)
        assert np.allclose(np.tril(got, -1) + np.eye(n), l, atol=1e-12)
        assert np.allclose(np.triu(got), u, atol=1e-10)


def test_oracle_reconstructs_the_matrix():
    a = _dominant(96, 7)
    got = ok.lud(a)
    l, u = np.tril(got, -1) + np.eye(96), np.triu(got)
    assert np.allclose(l @ u, a, atol=1e-10)


def test_coarsening_places_every_block_element_once():
    """The reference's ``inv``: virtual thread (ii, jj, tid) -> (i, j, tid/T, tid%T); with
    r = i*T + ty, c = j*T + tx the R*R*T*T virtual threads cover the block exactly once."""
    import sympy as sp
    ii, jj, tid = sp.symbols("ii jj tid", integer=True, nonnegative=True)
    f = sp.lambdify([ii, jj, tid], lud_gen.coarsening(ii, jj, tid), "math")
    T, R = lud_gen.T, lud_gen.R
    seen = set()
    for a in range(R):
        for b in range(R):
            for t in range(T * T):
                i, j, ty, tx = (int(v) for v in f(a, b, t))
                assert (i, j, ty, tx) == (a, b, t // T, t % T)
                seen.add((i * T + ty, j * T + tx))
    assert len(seen) == (R * T) ** 2


def _plan(n):
    """The launches of lego_hip_lud_f32 for an n x n matrix, as the library's own schedule records them."""
    import ctypes
    from lego_amd import runtime
    count = ctypes.c_int(0)
    runtime.call("lego_hip_lud_f32_plan", n, None, 0, ctypes.byref(count))
    buf = (ctypes.c_int * (6 * count.value))()
    runtime.call("lego_hip_lud_f32_plan", n, buf, count.value, ctypes.byref(count))
    return [tuple(buf[6 * i:6 * i + 6]) for i in range(count.value)]


def _replay(nb, plan):
    """Replays a recorded schedule on block indices: every launch finds its inputs final, every block gets each
    earlier step exactly once and in order, and what runs between a fork and the next join on the two streams
    touches disjoint blocks (write/write and read/write).  Returns how many forks there were."""
    applied = {(i, j): [] for i in range(nb) for j in range(nb)}
    solved = {}

    def update(block, steps, writes, reads):
        i, j = block
        assert block not in solved and block not in writes, block
        for st in steps:
            assert solved.get((i, st)) == st and solved.get((st, j)) == st, (block, st)
            applied[block].append(st)
            reads |= {(i, st), (st, j)}
        writes.add(block)

    forks, open_main, open_side = 0, None, None
    for kind, stream, a, b, c, d in plan:
        writes, reads = set(), set()
        if kind == 0:       # panels of step a, b workgroups
            assert b == nb - 1 - a
            assert applied[(a, a)] == list(range(a))
            reads.add((a, a))
            for w in range(b):
                for block in ((a, a + 1 + w), (a + 1 + w, a)):
                    assert applied[block] == list(range(a)) and block not in solved, block
                    solved[block] = a
                    writes.add(block)
        elif kind == 1:     # block row and column a+1 against step a
            assert b == nb - 1 - a
            for w in range(2 * b - 1):
                update((a + 1, a + 1 + w) if w < b else (a + 2 + w - b, a + 1), [a], writes, reads)
        elif kind == 2:     # two block rows and columns of the square of side c from block b on
            for w in range(4 * c - 4):
                block = (b + w // c, b + w % c) if w < 2 * c else (b + 2 + (w - 2 * c) // 2, b + (w - 2 * c) % 2)
                update(block, [a, a + 1], writes, reads)
        elif kind == 3:     # the square of side c from block b on
            depth, run = d // 16, d % 16
            assert run in (1, 2, 4, 8) and b + c == nb
            for i in range(c):
                for j in range(c):
                    update((b + i, b + j), list(range(a, a + depth)), writes, reads)
        elif kind == 4:
            assert open_main is None
            forks, open_main, open_side = forks + 1, (set(), set()), (set(), set())
            continue
        elif kind == 5:
            assert open_main is not None
            (mw, mr), (sw, sr) = open_main, open_side
            assert not (mw & sw) and not (mw & sr) and not (mr & sw)
            open_main = open_side = None
            continue
        else:
            assert kind == 6 and a == nb and open_main is None
            continue
        if open_main is None:
            assert stream == 0            # the side stream is only used between a fork and a join
        else:
            side = open_side if stream == 1 else open_main
            side[0].update(writes)
            side[1].update(reads)
    assert open_main is None and plan[-1][0] == 6
    for (i, j), steps in applied.items():
        assert steps == list(range(min(i, j))), (i, j)
    for i in range(nb):
        for j in range(nb):
            if i != j:
                assert solved[(i, j)] == min(i, j)
    return forks


@pytest.mark.parametrize("nb", list(range(1, 12)) + [63, 64, 76, 77, 78, 79, 100, 129, 256])
def test_launch_order_updates_every_block_in_order_and_overlaps_only_disjoint_work(nb):
    forks = _replay(nb, _plan(64 * nb))
    assert (forks > 0) == (nb >= lud_gen.AHEAD_MIN + 5)


def test_trailing_walk_covers_the_square_once():
    """The walk of the trailing update (groups of GROUP block rows, a column of a group in parts of `run` blocks)
    after the remap onto the XCDs: the layouts that print the kernel's index expressions, evaluated for every
    workgroup of the padded grid, give every block of a q x q square to exactly one workgroup, and one XCD
    (every XCDS-th workgroup id) gets a contiguous piece of the walk."""
    import sympy as sp
    ng, q, nsub, per, pid, wg = sp.symbols("ng q nsub per pid wg", integer=True, nonnegative=True)
    order = sp.lambdify([ng, q, nsub, pid], lud_gen.block_order(ng, q, nsub, pid), "math")
    remap = sp.lambdify([per, wg], lud_gen.xcd_remap(per, wg), "math")
    G, X = lud_gen.GROUP, lud_gen.XCDS
    for side in (1, 2, 7, 8, 9, 31, 64, 75, 124):
        for run in (1, 2, 4, 8):
            groups, parts = -(-side // G), G // run
            positions = groups * side * parts
            grid = -(-positions // X) * X
            seen, by_xcd = set(), {}
            for w in range(grid):
                pos = int(remap(grid // X, w))
                by_xcd.setdefault(w % X, []).append(pos)
                if pos >= positions:
                    continue
                g, c, part = (int(v) for v in order(groups, side, parts, pos))
                first = G * g + run * part
                for r in range(first, min(first + run, side)):
                    assert 0 <= c < side and (r, c) not in seen
                    seen.add((r, c))
            assert len(seen) == side * side, (side, run)
            for x, got in by_xcd.items():
                assert got == list(range(x * (grid // X), (x + 1) * (grid // X)))


@pytest.mark.gpu
@pytest.mark.parametrize("n", [64, 128, 512, 1024])
def test_gpu_matches_oracle(n):
    from lego_amd import ops
    print(f"lud n={n}", flush=True)
    a = _dominant(n, 100 + n).astype(np.float32)
    want = ok.lud(a)
    got = ops.lud(torch.from_numpy(a.copy()).cuda()).cpu().numpy().astype(np.float64)
    scale = np.abs(want).max()
    assert np.abs(got - want).max() <= 2e-5 * scale
    l, u = np.tril(got, -1) + np.eye(n), np.triu(got)
    assert np.abs(l @ u - a).max() <= 1e-4 * scale


@pytest.mark.gpu
def test_gpu_rejects_bad_sizes():
    from lego_amd import ops
    from lego_amd.runtime import LegoHipError
    with pytest.raises(LegoHipError):
        ops.lud(torch.eye(100, device="cuda"))


@pytest.mark.gpu
@pytest.mark.parametrize("n", [4928, 8256, 16384, 32768])
def test_gpu_large_matrix_reproduces_its_factors(n):
    """Sizes at which the panels of the next pair of steps are solved on a second stream (77 and 129 blocks: odd
    counts, the first the smallest that does), n = 16384, the largest size the reference publishes, and n = 32768, the
    largest the entry point takes (a 4 GiB matrix: offsets beyond 32 bits): L*U gives the
    matrix back (fp32, diagonally dominant)."""
    from lego_amd import ops
    print(f"lud n={n}", flush=True)
    a = torch.rand(n, n, device="cuda", generator=torch.Generator(device="cuda").manual_seed(61))
    a.diagonal().add_(float(n))
    w = a.clone()
    ops.lud(w)
    lower = torch.tril(w, -1)
    lower.diagonal().fill_(1.0)
    back = lower @ torch.triu(w)
    assert ((back - a).norm() / a.norm()).item() <= 1e-5


@pytest.mark.gpu
def test_gpu_call_with_second_stream_replays_from_a_hip_graph():
    """At n = 8256 the call forks to a second stream of the library and joins it back with events; captured into a
    graph on a stream that an eager call has used before (which made that stream's side stream), every replay
    gives the bits of the eager result, with eager work and synchronisation between the replays.  Captured on a
    stream the library has never seen, the call creates nothing and stays on the one stream: same bits."""
    from lego_amd import ops
    print("lud n=8256 captured into a graph", flush=True)
    n = 8256
    a = torch.rand(n, n, device="cuda", generator=torch.Generator(device="cuda").manual_seed(62))
    a.diagonal().add_(float(n))
    w = a.clone()
    ops.lud(w)
    torch.cuda.synchronize()
    want = w.clone()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        w.copy_(a)
        ops.lud(w)                       # warm-up on a side stream, outside the capture
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    for capture_stream in (side, torch.cuda.Stream()):      # known to the library / never seen by it
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=capture_stream):
            ops.lud(w)
        for trial in range(3):
            w.copy_(a)
            graph.replay()
            torch.cuda.synchronize()
            assert torch.equal(w, want), trial
            other = a[:512, :512] @ a[:512, :512]   # eager work between the replays
            torch.cuda.synchronize()
            del other
        del graph
