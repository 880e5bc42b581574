"""Pins of the oracle's helpers for 16-bit results: half_spacing against the element types' own
rounding, and the un-rounded LayerNorm against its definition in fp64."""
import pytest
import torch

from oracle import kernels as ok


@pytest.mark.parametrize("dtype,bits", [(torch.float16, 10), (torch.bfloat16, 7)])
def test_half_spacing_is_the_largest_rounding_error(dtype, bits):
    g = torch.Generator().manual_seed(0)
    y = torch.cat([3 * torch.randn(200000, generator=g), torch.tensor([1.0, 2.0, 3.999, 4.0, 1e-3, 0.0])])
    err = (y.to(dtype).float() - y).abs()
    hs = ok.half_spacing(y, dtype)
    assert (err <= hs).all()
    assert (err / hs).max().item() > 0.99          # and it is attained: the bound is tight
    # closed form at the binade ends: values in [2, 4) are 2^(1-bits) apart
    assert ok.half_spacing(torch.tensor([2.0, 3.999]), dtype).tolist() == [2.0 ** -bits, 2.0 ** -bits]
    assert ok.half_spacing(torch.tensor([4.0]), dtype).item() == 2.0 ** (1 - bits)


def test_unrounded_layernorm_is_the_definition():
    g = torch.Generator().manual_seed(1)
    x = (2 * torch.randn(7, 333, generator=g)).half()
    w = (1 + 0.1 * torch.randn(333, generator=g)).half()
    b = (0.1 * torch.randn(333, generator=g)).half()
    xd = x.double()
    mean = xd.mean(-1, keepdim=True)
    var = ((xd - mean) ** 2).mean(-1, keepdim=True)
    want = (xd - mean) / torch.sqrt(var + 1e-5) * w.double() + b.double()
    got = ok.layernorm_fwd_unrounded(x, w, b, 1e-5)
    assert got.dtype == torch.float32
    assert (got.double() - want).abs().max().item() <= 1e-5
    # and the rounded oracle is this value rounded
    assert torch.equal(ok.layernorm_fwd(x, w, b, 1e-5)[0], got.half())
