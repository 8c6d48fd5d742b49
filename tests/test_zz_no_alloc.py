"""mxq_reduce_outer_static -- the outer-axis reduction that allocates nothing (its partial results
live in a device array inside the library) -- against mxq_reduce_sum_outer / mxq_reduce_max_outer
with a caller-provided workspace, through the C ABI.  Same kernels and launch geometry, so the bits
must be the same; two calls in a row, the second on a smaller input, share the array."""
import ctypes

import pytest
import torch

from helpers import assert_bits_equal
from microxcaling_amd import _lib

pytestmark = pytest.mark.gpu


@pytest.fixture(autouse=True)
def need_gpu():
    assert torch.cuda.is_available(), "these tests need a GPU"

STATIC_BYTES = 16 << 20


def _stream():
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def _with_workspace(x, op):
    lib = _lib.gpu()
    outer, inner = x.shape
    n = lib.mxq_reduce_outer_workspace_bytes(outer, inner)
    ws = torch.empty(max(n, 16), dtype=torch.uint8, device=x.device)
    out = torch.empty(inner, dtype=torch.float32, device=x.device)
    fn = lib.mxq_reduce_max_outer if op else lib.mxq_reduce_sum_outer
    _lib.check(fn(x.data_ptr(), out.data_ptr(), ws.data_ptr(), outer, inner, _stream()), lib)
    return out, n


def _static(x, op, out):
    lib = _lib.gpu()
    outer, inner = x.shape
    _lib.check(lib.mxq_reduce_outer_static(x.data_ptr(), out.data_ptr(), op, outer, inner, _stream()), lib)
    return out


def test_static_scratch_reduction_equals_the_workspace_one_on_two_calls_in_a_row():
    g = torch.Generator().manual_seed(5)
    big = torch.randn(16384, 8192, generator=g)            # needs the whole 16 MiB array
    big[5, 7] = float("nan")
    big[9, 100] = float("inf")
    small = torch.randn(777, 1028, generator=g)            # fewer splits, shorter rows: stale partials around
    ragged = torch.randn(300, 1001, generator=g)           # one column per lane
    tiny = torch.randn(8, 64, generator=g)                 # a single split: no scratch at all
    for op in (0, 1):
        outs = []
        for x in (big, small, ragged, tiny):
            xd = x.cuda()
            outs.append((xd, torch.empty(xd.shape[1], dtype=torch.float32, device="cuda")))
        for xd, out in outs:                               # back to back on one stream, no sync between
            _static(xd, op, out)
        torch.cuda.synchronize()
        for xd, out in outs:
            want, need = _with_workspace(xd, op)
            assert need <= STATIC_BYTES
            torch.cuda.synchronize()
            assert_bits_equal(out.cpu(), want.cpu(), "op %d shape %s" % (op, tuple(xd.shape)))
            ref = xd.max(0).values if op else xd.double().sum(0)
            if op:
                assert_bits_equal(out.cpu(), ref.cpu(), "max vs torch")
            else:
                fin = torch.isfinite(ref)
                tol = 1e-5 * xd.double().abs().sum(0)
                assert torch.equal(torch.isnan(out.double()), torch.isnan(ref))
                assert bool(((out.double() - ref).abs()[fin] <= tol[fin]).all())


def test_static_scratch_reduction_refuses_what_does_not_fit():
    lib = _lib.gpu()
    outer, inner = 65536, 3 * 1024                         # ceil(4096 / 3) splits of 3072 columns: just over
    assert lib.mxq_reduce_outer_workspace_bytes(outer, inner) > STATIC_BYTES
    x = torch.empty(outer, inner, device="cuda")
    out = torch.full((inner,), 3.0, device="cuda")
    rc = lib.mxq_reduce_outer_static(x.data_ptr(), out.data_ptr(), 0, outer, inner, _stream())
    assert rc != 0 and b"scratch" in lib.mxq_last_error()
    assert lib.mxq_reduce_outer_static(x.data_ptr(), out.data_ptr(), 2, 8, 8, _stream()) != 0
    torch.cuda.synchronize()
    assert bool((out == 3.0).all())                        # nothing was launched
