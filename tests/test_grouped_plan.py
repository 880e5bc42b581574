"""The launch that lego_hip_grouped_gemm_f16 makes, replayed on the host: the plan the entry point
reports, the workgroup -> (problem, tile, half) map of the kernels (the LEGO layouts the generator
prints into them, evaluated with integers), and that the workgroups' blocks of C tile every problem
exactly once."""
import ctypes

import numpy as np
import pytest

from lego_amd import runtime
from lego_amd.kernels import gemm
from lego_amd.lego import OrderBy, Row

C5 = [(4096, 1024, 2048), (1024, 4096, 2048), (2048, 4096, 1024), (2048, 2048, 1024), (4096, 4096, 1024),
      (1024, 1024, 1024), (4096, 2048, 1024), (1024, 1024, 1024)]


def _plan(sizes):
    sz = (ctypes.c_int * (3 * len(sizes)))(*[v for s in sizes for v in s])
    out = (ctypes.c_int * 3)()
    runtime.call("lego_hip_grouped_gemm_f16_plan", sz, len(sizes), out)
    return list(out)


def _group_height(num_pid_m, max_gm=8):
    gm = max_gm
    while num_pid_m % gm:
        gm -= 1
    return gm


def _coverage(sizes, split):
    """Blocks of 128 x 256 of every problem's C, counted over all workgroups of the split launch."""
    order = sorted(range(len(sizes)), key=lambda g: -sizes[g][2])        # decreasing depth, stable
    tiles = [(-(-sizes[g][0] // 256), -(-sizes[g][1] // 256)) for g in order]
    ends = np.cumsum([tm * tn for tm, tn in tiles])
    total = int(ends[-1])
    whole = total - split
    seen = [np.zeros((2 * tm, tn), dtype=int) for tm, tn in tiles]
    depth = [sizes[g][2] for g in order]

    def depth_class(tile):
        """Flat tile range of the problems whose depth is that of the problem holding `tile`."""
        s = int(np.searchsorted(ends, tile, side="right"))
        first = min(q for q in range(len(order)) if depth[q] == depth[s])
        last = max(q for q in range(len(order)) if depth[q] == depth[s])
        return (int(ends[first - 1]) if first else 0), int(ends[last])

    for wg in range(total + split):
        if wg < whole:
            cb, ce = depth_class(wg)
            tile, half = cb + gemm.class_order(wg - cb, min(ce, whole) - cb, cb), None
        else:
            cb, ce = depth_class(whole + (wg - whole) // 2)
            first_tile = max(cb, whole)
            first_wg = whole + 2 * (first_tile - whole)
            swg = gemm.class_order(wg - first_wg, 2 * (ce - first_tile), first_wg)
            t, half = gemm.split_order(ce - first_tile, swg)            # Row(tiles, 2).inv(swg)
            tile = first_tile + int(t)
        s = int(np.searchsorted(ends, tile, side="right"))
        pid = tile - (int(ends[s - 1]) if s else 0)
        npm, npn = tiles[s]
        pid_m, pid_n = (int(v) for v in gemm.launch_order(npm, npn, _group_height(npm), pid))
        assert 0 <= pid_m < npm and 0 <= pid_n < npn
        if half is None:
            seen[s][2 * pid_m:2 * pid_m + 2, pid_n] += 1
        else:
            half_m = int(OrderBy(Row(npm, 2)).TileBy([npm, 2])[pid_m, int(half)])
            seen[s][half_m, pid_n] += 1
    return seen, total


@pytest.mark.parametrize("sizes", [C5, [(256, 256, 64)], [(1000, 776, 192), (520, 264, 128), (136, 512, 64)],
                                   [(2048, 2048, 512)] * 5, [(4096, 4096, 4096), (512, 512, 64)],
                                   [(768, 256, 192), (4352, 4352, 128), (1024, 1280, 128), (2048, 2304, 64),
                                    (1536, 1024, 64)]])
def test_every_block_of_c_is_computed_once(sizes):
    kind, total, split = _plan(sizes)
    assert total == sum(-(-m // 256) * -(-n // 256) for m, n, _ in sizes)
    assert 0 <= split <= total
    for s in sorted({0, 1, split, total // 2, total}):
        seen, _ = _coverage(sizes, s)
        for blocks in seen:
            assert (blocks == 1).all()


def test_plan_splits_the_tail_of_the_headline_problem_set():
    kind, total, split = _plan(C5)
    # 128 tiles of depth 32 and 608 of depth 16 on 256 CUs: three rounds and 96 tiles over; the
    # plan gives that tail (or more) to halves
    assert (kind, total) == (256, 736) and 96 <= split <= 224 and split % 16 == 0


def test_plan_keeps_whole_rounds_whole_and_small_sets_on_small_tiles():
    assert _plan([(4096, 4096, 1024)]) == [256, 256, 0]            # exactly one round of whole tiles
    assert _plan([(8192, 8192, 2048)])[2] == 0                     # four rounds
    assert _plan([(1024, 512, 256), (512, 512, 512)])[0] == 128    # a handful of tiles: 128 x 128 tiles
    with pytest.raises(runtime.LegoHipError):
        _plan([(0, 256, 64)])


def _gemm_plan(M, N, K=4096):
    out = (ctypes.c_int * 2)()
    runtime.call("lego_hip_gemm_plan", M, N, K, out)
    return tuple(out)


def test_gemm_plan_follows_the_measured_crossovers():
    """The single-product dispatch, on the host: (tile side, MFMA block side) for the shapes its thresholds were
    measured on."""
    big, small, sparse = (256, 16), (128, 32), (256, 32)
    assert _gemm_plan(8192, 8192) == big and _gemm_plan(4096, 4096) == big          # whole rounds
    assert _gemm_plan(2048, 2048) == small and _gemm_plan(2048, 4096) == small        # up to 128 big tiles
    # one round that leaves a third of the CUs idle: the 32x32x16 build up to 175 tiles
    assert _gemm_plan(3072, 3072) == sparse and _gemm_plan(2304, 4096) == sparse and _gemm_plan(2560, 4096) == sparse
    assert _gemm_plan(2816, 4096) == big and _gemm_plan(3584, 3584) == big
    # a mostly empty second round: small tiles while they make the estimate in rounds shorter
    assert _gemm_plan(4352, 4096) == small and _gemm_plan(5120, 4096) == small and _gemm_plan(4608, 4608) == small
    assert _gemm_plan(6144, 4096) == big and _gemm_plan(5120, 5120) == big and _gemm_plan(6144, 6144) == big
    assert _gemm_plan(7168, 4096) == big
    # ragged tiles count as whole ones
    assert _gemm_plan(3071, 3065) == sparse and _gemm_plan(8184, 8184) == big
    with pytest.raises(runtime.LegoHipError):
        _gemm_plan(0, 256)


def _rows_plan(M, N):
    out = ctypes.c_int()
    runtime.call("lego_hip_rows_f16_plan", M, N, ctypes.byref(out))
    return out.value


def test_row_team_sizes_follow_the_measured_crossovers():
    """Waves per row of the fp16 softmax and LayerNorm forward, on the host, for the shapes the thresholds were
    measured on."""
    assert _rows_plan(8192, 8192) == 8 and _rows_plan(8192, 16384) == 8 and _rows_plan(8192, 6152) == 8    # long rows, tall
    assert _rows_plan(2048, 8192) == 4 and _rows_plan(8192, 6144) == 4 and _rows_plan(8192, 4096) == 4
    assert _rows_plan(4096, 4096) == 2 and _rows_plan(2500, 3080) == 2        # one round of workgroups instead of two
    assert _rows_plan(8192, 2048) == 1 and _rows_plan(65536, 1024) == 1 and _rows_plan(32768, 1536) == 1
    assert _rows_plan(16384, 2048) == 2 and _rows_plan(65536, 1600) == 2      # four vectors per lane of one wave, very tall
    assert _rows_plan(512, 32768) == 16 and _rows_plan(600, 20488) == 16
    for bad in ((8192, 8191), (0, 8), (8, 32776)):
        with pytest.raises(runtime.LegoHipError):
            _rows_plan(*bad)
