"""The CPU baseline's path: offsets printed by the Python/Triton printer, evaluated with torch.arange,
against the oracle's integer layouts and the textbook transpose; and the benchmark's reading of the
committed HBM-traffic summary."""
import numpy as np
import pytest
import torch

from lego_amd.kernels.transpose import python_offsets
from oracle import cpu_path
from oracle import kernels as ok
from oracle import lego_index as li


@pytest.mark.parametrize("rows,cols,tr,tc", [(256, 384, 64, 64), (128, 128, 32, 32), (96, 160, 32, 16)])
def test_printed_offsets_are_the_oracle_layouts(rows, cols, tr, tc):
    src_text, dst_text = python_offsets(tr, tc)
    names = dict(R=rows, C=cols, nbi=rows // tr, nbj=cols // tc)
    src, dst = ok.transpose_layouts(rows, cols, tr, tc)
    assert np.array_equal(cpu_path.evaluate(src_text, **names).numpy(), np.array(src.offsets()))
    assert np.array_equal(cpu_path.evaluate(dst_text, **names).numpy(), np.array(dst.offsets()))
    # closed forms of the two layouts: r*C + c and c*R + r
    bi, bj, i, j = np.meshgrid(np.arange(rows // tr), np.arange(cols // tc), np.arange(tr), np.arange(tc), indexing="ij")
    assert np.array_equal(cpu_path.evaluate(src_text, **names).numpy(), (bi * tr + i) * cols + bj * tc + j)
    assert np.array_equal(cpu_path.evaluate(dst_text, **names).numpy(), (bj * tc + j) * rows + bi * tr + i)


def test_cpu_path_transposes_whole_matrices_and_panels():
    g = torch.Generator().manual_seed(0)
    src_text, dst_text = python_offsets(64, 64)
    x = torch.randn(256, 384, generator=g).half()
    assert torch.equal(cpu_path.transpose_printed(x, src_text, dst_text, 64, 64), x.t().contiguous())
    assert torch.equal(cpu_path.transpose_printed(x, src_text, dst_text, 64, 64), ok.transpose(x, 64, 64))
    got = cpu_path.transpose_printed(x[:128], src_text, dst_text, 64, 64, total_rows=256)
    assert torch.equal(got, x.t()[:, :128].contiguous())


def test_benchmark_reads_the_committed_traffic_summary():
    import bench
    got = bench.headline_traffic_bytes()
    text = open(bench.TRAFFIC_PROFILE).read()
    row = next(line for line in text.splitlines() if line.startswith((bench.HEADLINE_KERNEL + " ", bench.HEADLINE_KERNEL + "<")))
    fetch_kib, write_kib, scaled, algorithmic = [int(t) for t in row.split(")", 1)[1].split()[:4]]
    assert got == scaled
    # the scaled figure is what the counters say, each scaled by what the same counter reads for the plain
    # 512 MiB copy in the same file (FETCH_SIZE counts half of every 128-byte request at this access width)
    import re
    cal_fetch, cal_write = (int(v) for v in re.search(r"reads FETCH_SIZE=(\d+) KiB and writes WRITE_SIZE=(\d+) KiB", text).groups())
    known = 512 * 1024
    assert abs(scaled - (known / cal_fetch * fetch_kib + known / cal_write * write_kib) * 1024) <= 4096
    assert algorithmic == 2 * 16384 * 16384 * 2
