"""The ctypes replacement for the reference's mx/custom_extensions.py that INTEGRATION.md prints, run as code
on the GPU: its five GPU functions against the oracle (the two CPU ones: tests/test_api_surface.py)."""
import pytest
import torch

from helpers import assert_bits_equal, integration_stub


@pytest.mark.gpu
def test_the_reference_side_stub_on_the_gpu():
    from oracle import mx_oracle as O
    assert torch.cuda.is_available(), "this test needs a GPU"
    stub = integration_stub()
    g = torch.Generator().manual_seed(6)
    x = torch.randn(64, 256, generator=g) * 3
    xd = x.cuda()
    got = stub.funcs.quantize_mx_by_tile_func_cuda(xd, 8, 4, 5, 448.0, 32, 1, False, 0)
    assert_bits_equal(got.cpu(), O.quantize_mx(x, 8, "fp8_e4m3", axes=[-1], block_size=32), "by tile")
    blocks = xd.view(64, 8, 32)
    got = stub.funcs.quantize_mx_func_cuda(blocks, 8, 4, 5, 448.0, blocks.abs().max(dim=2, keepdim=True).values, 2)
    assert_bits_equal(got.cpu().view(64, 256), O.quantize_mx(x, 8, "fp8_e4m3", axes=[-1], block_size=32), "given max")
    got = stub.funcs.quantize_elemwise_func_cuda(xd, 9, 8, 2 ** 127 * 255 / 128, 0, False, True)
    assert_bits_equal(got.cpu(), O.quantize_elemwise_core(x, 9, 8, 2 ** 127 * 255 / 128), "elementwise")
    assert torch.equal(stub.funcs.reduce_max_inner_dim(xd).cpu(), x.max(dim=-1).values)
    s = stub.funcs.reduce_sum_inner_dim(xd).cpu()
    assert bool(((s - x.double().sum(-1).float()).abs() <= 1e-5 * x.abs().sum(-1)).all())
