"""The reference's transpose programs, generated through the HIP kernel builder, run on
the GPU and are bit exact (the reference itself never checks them:
benchmarks/mlir/transpose_smem.py:82-83 is commented out)."""
import pytest
import torch

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("n", [256, 1024])
@pytest.mark.parametrize("kind", ["naive", "smem"])
def test_dsl_transpose(kind, n):
    print(f"dsl transpose {kind} {n}", flush=True)
    from lego_amd.kernels.dsl_transpose import transpose_naive, transpose_smem
    mod = (transpose_naive if kind == "naive" else transpose_smem)(n)
    assert mod.so_path.exists(), "builder-DSL modules are compiled by __graft_entry__.build()"
    x = torch.arange(n * n, dtype=torch.float32).view(n, n).cuda()   # the reference's fill: element k = k
    y = torch.empty_like(x)
    mod.launch(mod.launchers[0], x, y, stream=torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    assert torch.equal(y, x.t())


def test_dsl_loop_carried_row_sums():
    print("dsl row sums", flush=True)
    from lego_amd.kernels.dsl_transpose import row_sums
    mod = row_sums(256, 96)
    assert mod.so_path.exists(), "builder-DSL modules are compiled by __graft_entry__.build()"
    x = torch.randint(-8, 9, (256, 96), generator=torch.Generator().manual_seed(0)).float().cuda()   # exact sums
    y = torch.empty(256, device="cuda")
    mod.launch(mod.launchers[0], x, y, stream=torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    assert torch.equal(y, x.sum(1))
