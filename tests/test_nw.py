"""Needleman-Wunsch: the oracle is pinned on the CPU, the kernel against the oracle on the GPU."""
import numpy as np
import pytest
import sympy as sp
import torch

from lego_amd.kernels import nw
from oracle import kernels as ok


def _loops(ref, penalty):
    n1 = ref.shape[0]
    m = [[0] * n1 for _ in range(n1)]
    for i in range(n1):
        m[i][0] = -i * penalty
        m[0][i] = -i * penalty
    for i in range(1, n1):
        for j in range(1, n1):
            m[i][j] = max(m[i - 1][j - 1] + int(ref[i, j]), m[i][j - 1] - penalty, m[i - 1][j] - penalty)
    return np.array(m, dtype=np.int32)


def test_oracle_matches_the_plain_double_loop():
    rng = np.random.default_rng(0)
    for n, penalty in ((7, 10), (16, 3), (33, 1)):
        ref = rng.integers(-4, 12, size=(n + 1, n + 1)).astype(np.int32)
        assert np.array_equal(ok.needleman_wunsch(ref, penalty), _loops(ref, penalty))


def test_oracle_closed_form_without_substitution_scores():
    """With zero scores a diagonal step is free and a gap costs ``penalty``: m[i][j] = -|i-j|*penalty."""
    n = 40
    got = ok.needleman_wunsch(np.zeros((n + 1, n + 1), dtype=np.int32), 7)
    i, j = np.meshgrid(np.arange(n + 1), np.arange(n + 1), indexing="ij")
    assert np.array_equal(got, -np.abs(i - j) * 7)


def test_rotation_through_lds_is_free_of_bank_conflicts():
    """Slot k of lane tx is row (k - tx) mod 64 of column tx: in the kernel's LDS tile the 64 lanes
    of every such access, and of every row access, fall into 64 different banks."""
    b = nw.B
    i, j = sp.symbols("i j", integer=True, nonnegative=True)
    f = sp.lambdify([i, j], nw.rotation_layout()[i, j], "math")
    words = set()
    for k in range(b):
        slots = [int(f((k - tx) % b, tx)) for tx in range(b)]
        assert len({w % 64 for w in slots}) == 64
        words.update(slots)
        assert len({int(f(k, tx)) % 64 for tx in range(b)}) == 64
    assert words == set(range(b * b))


def test_tile_layout_is_the_anti_diagonal_enumeration():
    """The reference's layout of the tile (nw_sympy.py:9-11): a bijection of the 64 x 64 tile in
    which the cells of one anti-diagonal are consecutive and ordered by row."""
    b = nw.B
    i, j = sp.symbols("i j", integer=True, nonnegative=True)
    f = sp.lambdify([i, j], nw.tile_layout()[i, j], "math")
    table = np.array([[int(f(a, c)) for c in range(b)] for a in range(b)])
    assert sorted(table.ravel().tolist()) == list(range(b * b))
    pos = 0
    for d in range(2 * b - 1):
        for a in range(max(0, d - b + 1), min(d, b - 1) + 1):
            assert table[a, d - a] == pos
            pos += 1


@pytest.mark.gpu
@pytest.mark.parametrize("n,penalty", [(64, 10), (256, 10), (1024, 3), (2048, 10)])
def test_gpu_matches_oracle(n, penalty):
    from lego_amd import ops
    print(f"needleman-wunsch n={n} penalty={penalty}", flush=True)
    g = torch.Generator().manual_seed(20 + n)
    ref = torch.randint(-4, 12, (n + 1, n + 1), generator=g, dtype=torch.int32)
    want = torch.from_numpy(ok.needleman_wunsch(ref.numpy(), penalty))
    m = torch.zeros((n + 1, n + 1), dtype=torch.int32)
    m[:, 0] = -torch.arange(n + 1, dtype=torch.int32) * penalty
    m[0, :] = -torch.arange(n + 1, dtype=torch.int32) * penalty
    got = ops.needleman_wunsch(ref.cuda(), m.cuda(), penalty).cpu()
    assert torch.equal(got, want)


@pytest.mark.gpu
def test_gpu_rejects_bad_sizes():
    from lego_amd import ops
    from lego_amd.runtime import LegoHipError
    with pytest.raises(LegoHipError):
        ops.needleman_wunsch(torch.zeros(101, 101, dtype=torch.int32, device="cuda"),
                             torch.zeros(101, 101, dtype=torch.int32, device="cuda"), 10)


@pytest.mark.gpu
def test_gpu_maximum_size_closed_form():
    """The largest size the entry point takes, n = 32768: with zero scores a diagonal step is free and a
    gap costs the penalty, so m[i][j] = -|i - j| * penalty."""
    from lego_amd import ops
    print("needleman-wunsch n=32768, zero scores", flush=True)
    n, penalty = 32768, 3
    ref = torch.zeros((n + 1, n + 1), dtype=torch.int32, device="cuda")
    m = torch.zeros((n + 1, n + 1), dtype=torch.int32, device="cuda")
    border = -torch.arange(n + 1, dtype=torch.int32, device="cuda") * penalty
    m[0, :] = border
    m[:, 0] = border
    ops.needleman_wunsch(ref, m, penalty)
    idx = torch.arange(n + 1, device="cuda", dtype=torch.int32)
    for rows in (slice(0, 130), slice(16000, 16130), slice(n - 129, n + 1)):
        want = -(idx[rows, None] - idx[None, :]).abs() * penalty
        assert torch.equal(m[rows], want)
