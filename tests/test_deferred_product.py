"""mx.bmm's deferred product (bmm.DeferredProduct): mx.softmax(mx.bmm(q, k^T), dim=-1) -- the reference's own
call sequence for attention scores (mx/bmm.py:138-145, mx/softmax.py:91-97) -- reaches the one-launch
product + softmax kernel, and everything else that touches the product sees the tensor mx.bmm would have
returned.  The laziness itself is device independent and is tested here on CPU tensors (the product is then
evaluated by the host library); the GPU cases check the kernels behind it through the C ABI."""
import pytest
import torch

from helpers import assert_bits_equal


def _specs(**kw):
    from microxcaling_amd.specs import finalize_mx_specs
    return finalize_mx_specs(dict(kw), early_exit=False)


def _operands(batch=3, M=40, N=64, K=128, seed=0):
    g = torch.Generator().manual_seed(seed)
    q = torch.randn(batch, M, K, generator=g).to(torch.bfloat16)
    k = torch.randn(batch, N, K, generator=g).to(torch.bfloat16)
    return q, k.transpose(-1, -2)


SPECS = dict(a_elem_format="fp6_e2m3", block_size=32, bfloat=16)


def test_a_deferred_product_behaves_like_the_product():
    from microxcaling_amd.bmm import DeferredProduct, bmm
    from microxcaling_amd.softmax import softmax
    specs = _specs(**SPECS)
    q, kt = _operands()
    want = bmm(q, kt, mx_specs=specs)                           # CPU operands: evaluated at once
    assert type(want) is torch.Tensor
    d = DeferredProduct(q, kt, specs, None)
    assert d.shape == want.shape and d.dtype == want.dtype and d.device == want.device and d.dim() == 3
    assert d.pending() is not None and "pending" in repr(d)
    assert_bits_equal(d + 0, want, "first use evaluates the product")
    assert d.pending() is None and "evaluated" in repr(d)
    assert_bits_equal(d[1, :5], want[1, :5], "indexing")
    assert_bits_equal(d.float().to(torch.bfloat16), want, "casts")
    assert d.data_ptr() == d.materialize().data_ptr() != 0
    # in place: the object the caller holds is the modified product from then on
    d2, ref = DeferredProduct(q, kt, specs, None), want.clone()
    mask = torch.zeros_like(want)
    mask[:, :, 10:] = float("-inf")
    d2.add_(mask)
    ref.add_(mask)
    assert_bits_equal(d2 * 1, ref, "in place")
    assert_bits_equal(softmax(d2, dim=-1, mx_specs=specs), softmax(ref, dim=-1, mx_specs=specs), "softmax after a mask")
    # the softmax of a pending product, where the one-launch kernel does not apply (CPU): the two steps
    d3 = DeferredProduct(q, kt, specs, None)
    assert_bits_equal(softmax(d3, dim=-1, mx_specs=specs), softmax(want, dim=-1, mx_specs=specs), "softmax, two steps")
    assert_bits_equal(softmax(DeferredProduct(q, kt, specs, None), dim=1, mx_specs=specs),
                      softmax(want, dim=1, mx_specs=specs), "another axis")
    # as an operand of the next product
    v = torch.randn(3, 64, 128, generator=torch.Generator().manual_seed(1)).to(torch.bfloat16)
    assert_bits_equal(bmm(DeferredProduct(q, kt, specs, None), v, mx_specs=specs), bmm(want, v, mx_specs=specs), "bmm of it")


def test_a_pending_product_goes_to_the_one_launch_kernel(monkeypatch):
    """With the kernel's conditions met (stand-ins here: no GPU), mx.softmax over the last axis hands the
    operands over once and never evaluates the product; other specs, another axis or an evaluated product
    do not take that path."""
    import importlib
    B = importlib.import_module("microxcaling_amd.bmm")         # the package exports the function under this name
    from microxcaling_amd.softmax import softmax
    specs = _specs(**SPECS)
    q, kt = _operands()
    calls = []

    def stand_in(in1, in2, sp):
        calls.append((in1, in2))
        return torch.full(in1.shape[:-1] + (in2.shape[-1],), 0.5, dtype=in1.dtype)
    monkeypatch.setattr(B, "_scores_in_one_launch", stand_in)
    d = B.DeferredProduct(q, kt, specs, None)
    out = softmax(d, dim=-1, mx_specs=specs)
    assert len(calls) == 1 and calls[0][0] is q and calls[0][1] is kt and bool((out == 0.5).all())
    assert d.pending() is not None                               # the product itself was never needed
    softmax(d, dim=2, mx_specs=specs)
    assert len(calls) == 2
    softmax(d, dim=1, mx_specs=specs)                            # not the last axis
    assert len(calls) == 2 and d.pending() is None
    softmax(d, dim=-1, mx_specs=specs)                           # evaluated by now
    assert len(calls) == 2
    other = _specs(a_elem_format="fp6_e2m3", block_size=32, bfloat=16, softmax_exp2=True)
    d = B.DeferredProduct(q, kt, specs, None)
    softmax(d, dim=-1, mx_specs=other)                           # a softmax under other specs than the product's
    assert len(calls) == 2 and d.pending() is None


def test_the_softmax_module_and_injected_names_meet_a_pending_product_too(monkeypatch):
    """mx.Softmax (what inject_pyt_ops binds torch.nn.Softmax to) takes the same path as mx.softmax: a layer that
    called the autograd function directly would evaluate the product and never reach the one-launch kernel."""
    import importlib
    B = importlib.import_module("microxcaling_amd.bmm")
    from microxcaling_amd.softmax import Softmax
    specs = _specs(**SPECS)
    q, kt = _operands()
    calls = []

    def stand_in(in1, in2, sp):
        calls.append(1)
        return torch.full(in1.shape[:-1] + (in2.shape[-1],), 0.25, dtype=in1.dtype)
    monkeypatch.setattr(B, "_scores_in_one_launch", stand_in)
    d = B.DeferredProduct(q, kt, specs, None)
    out = Softmax(dim=-1, mx_specs=specs)(d)
    assert calls == [1] and d.pending() is not None and bool((out == 0.25).all())


def test_modifying_an_operand_before_the_product_is_used_raises():
    from microxcaling_amd.bmm import DeferredProduct
    specs = _specs(**SPECS)
    q, kt = _operands()
    d = DeferredProduct(q, kt, specs, None)
    q.mul_(2.0)
    with pytest.raises(RuntimeError, match="modified in place"):
        d + 0


def test_cpu_and_switched_off_products_are_evaluated_at_once():
    from microxcaling_amd import gemm
    from microxcaling_amd.bmm import bmm
    specs = _specs(**SPECS)
    q, kt = _operands()
    assert type(bmm(q, kt, mx_specs=specs)) is torch.Tensor
    assert gemm.deferred_scores_enabled()
    gemm.set_deferred_scores(False)
    try:
        assert not gemm.deferred_scores_enabled()
    finally:
        gemm.set_deferred_scores(True)
