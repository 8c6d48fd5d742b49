"""Forward outputs and gradients of the MX layers against fixtures written by the reference's own
CPU path (tests/golden/gen_reference_layer_vectors.py): the oracle's restatements, and the
package's layers on CPU tensors (host library quantizers + torch's GEMM).  Bit for bit -- same
torch, same op order, single-threaded GEMM."""
import os

import numpy as np
import pytest
import torch

from helpers import ROOT_DIR, assert_bits_equal
from oracle import mx_oracle as O

FIX = np.load(os.path.join(ROOT_DIR, "tests", "golden", "reference_layer_vectors.npz"))


def fx(name):
    if name + ":bf16" in FIX:
        return torch.from_numpy(FIX[name + ":bf16"].copy()).view(torch.bfloat16)
    return torch.from_numpy(FIX[name + ":f32"].copy()).view(torch.float32)


@pytest.fixture(autouse=True)
def one_thread():
    n = torch.get_num_threads()
    torch.set_num_threads(1)
    yield
    torch.set_num_threads(n)


DT = {"f32": torch.float32, "bf16": torch.bfloat16}


def _specs(**kw):
    from microxcaling_amd.specs import finalize_mx_specs
    return finalize_mx_specs(dict(kw))


@pytest.mark.parametrize("dt", ["f32", "bf16"])
@pytest.mark.parametrize("bfloat", [0, 16])
def test_linear_oracle_and_cpu_layer(dt, bfloat):
    x, w, b, go = (fx("in/" + n).to(DT[dt]) for n in ("x", "w", "b", "go"))
    key = "linear/%s/bfloat%d/" % (dt, bfloat)
    out = O.mx_linear_forward(x, w, b, "fp8_e4m3", "fp8_e4m3", bfloat=bfloat)
    assert_bits_equal(out, fx(key + "out"), "oracle forward")
    gi, gw, gb = O.mx_linear_backward(x, w, go, True, "fp8_e4m3", bfloat=bfloat)
    assert_bits_equal(gi, fx(key + "gx"), "oracle grad_input")
    assert_bits_equal(gw, fx(key + "gw"), "oracle grad_weight")
    assert_bits_equal(gb, fx(key + "gb"), "oracle grad_bias")

    from microxcaling_amd.linear import linear
    specs = _specs(w_elem_format="fp8_e4m3", a_elem_format="fp8_e4m3", block_size=32, bfloat=bfloat,
                   quantize_backprop=True)
    xi, wi, bi = (t.clone().requires_grad_(True) for t in (x, w, b))
    o = linear(xi, wi, bi, mx_specs=specs)
    o.backward(go)
    assert_bits_equal(o.detach(), fx(key + "out"), "layer forward")
    assert_bits_equal(xi.grad, fx(key + "gx"), "layer grad_input")
    assert_bits_equal(wi.grad, fx(key + "gw"), "layer grad_weight")
    assert_bits_equal(bi.grad, fx(key + "gb"), "layer grad_bias")


def test_linear_with_prequantized_weights():
    """mx/linear.py:246-274: weight and bias stored as bf16 once (round-half-even), inference on bf16
    inputs and on fp32 inputs (mx/linear.py:77-80).  On CPU tensors no packed form is built."""
    from microxcaling_amd.linear import Linear
    x, w, b = fx("in/x"), fx("in/w"), fx("in/b")
    specs = _specs(w_elem_format="fp8_e4m3", a_elem_format="fp8_e4m3", block_size=32, bfloat=16, round="even")
    m = Linear(64, 48, bias=True, mx_specs=specs)
    with torch.no_grad():
        m.weight.copy_(w)
        m.bias.copy_(b)
    m.prequantize_weights()
    m.eval()
    assert m.weight.dtype == torch.bfloat16 and m.bias.dtype == torch.bfloat16
    assert_bits_equal(m.weight.data, fx("linear_prequantized/p_weight"), "stored weight")
    assert_bits_equal(m.bias.data, fx("linear_prequantized/p_bias"), "stored bias")
    with torch.no_grad():
        assert_bits_equal(m(x.to(torch.bfloat16)), fx("linear_prequantized/out_bf16"), "bf16 input")
        assert_bits_equal(m(x), fx("linear_prequantized/out_f32"), "fp32 input")
    assert m.packed_weight_bytes() == 0
    m.train()
    with pytest.raises(AssertionError, match="prequantized weights when training"):
        m(x)
    # a layer without MX specs has nothing to prequantize
    plain = Linear(64, 48, mx_specs=None)
    plain.prequantize_weights()
    assert plain.weight.dtype == torch.float32 and not plain.prequantized_weights
    # the reference's preconditions
    with pytest.raises(AssertionError, match="'even'"):
        Linear(64, 48, mx_specs=_specs(w_elem_format="fp8_e4m3", a_elem_format="fp8_e4m3", block_size=32,
                                       bfloat=16, round="nearest")).prequantize_weights()


@pytest.mark.parametrize("block", [64, 0])
def test_linear_blocks_that_do_not_divide_the_example_axis(block):
    """3-D input (3, 96, 64) with block size 64 or "whole axis": the weight gradient's exponents
    are shared along the example axis of each batch entry (mx/linear.py:124-143), never across
    entries."""
    x, go, w, b = fx("in/x3"), fx("in/go3"), fx("in/w"), fx("in/b")
    key = "linear_block%d/" % block
    out = O.mx_linear_forward(x, w, b, "fp8_e4m3", "fp8_e4m3", block_size=block, bfloat=16)
    assert_bits_equal(out, fx(key + "out"), "oracle forward")
    gi, gw, gb = O.mx_linear_backward(x, w, go, True, "fp8_e4m3", block_size=block, bfloat=16)
    assert_bits_equal(gi, fx(key + "gx"), "oracle grad_input")
    assert_bits_equal(gw, fx(key + "gw"), "oracle grad_weight")
    assert_bits_equal(gb, fx(key + "gb"), "oracle grad_bias")

    from microxcaling_amd.linear import linear
    specs = _specs(w_elem_format="fp8_e4m3", a_elem_format="fp8_e4m3", block_size=block, bfloat=16,
                   quantize_backprop=True)
    xi, wi, bi = (t.clone().requires_grad_(True) for t in (x, w, b))
    o = linear(xi, wi, bi, mx_specs=specs)
    o.backward(go)
    assert_bits_equal(o.detach(), fx(key + "out"), "layer forward")
    assert_bits_equal(xi.grad, fx(key + "gx"), "layer grad_input")
    assert_bits_equal(wi.grad, fx(key + "gw"), "layer grad_weight")
    assert_bits_equal(bi.grad, fx(key + "gb"), "layer grad_bias")


@pytest.mark.parametrize("dt", ["f32", "bf16"])
def test_bmm_oracle_and_cpu_layer(dt):
    a, b, go = (fx("in/" + n).to(DT[dt]) for n in ("x", "a2", "go2"))
    key = "bmm/%s/" % dt
    assert_bits_equal(O.mx_bmm_forward(a, b, "fp6_e2m3"), fx(key + "out"), "oracle forward")
    g1, g2 = O.mx_bmm_backward(a, b, go, "fp6_e2m3")
    assert_bits_equal(g1, fx(key + "g1"), "oracle grad_in1")
    assert_bits_equal(g2, fx(key + "g2"), "oracle grad_in2")

    from microxcaling_amd.bmm import bmm
    specs = _specs(a_elem_format="fp6_e2m3", block_size=32, quantize_backprop=True)
    ai, bi = a.clone().requires_grad_(True), b.clone().requires_grad_(True)
    o = bmm(ai, bi, mx_specs=specs)
    o.backward(go)
    assert_bits_equal(o.detach(), fx(key + "out"), "layer forward")
    assert_bits_equal(ai.grad, fx(key + "g1"), "layer grad_in1")
    assert_bits_equal(bi.grad, fx(key + "g2"), "layer grad_in2")


@pytest.mark.parametrize("dt", ["f32", "bf16"])
@pytest.mark.parametrize("case", ["2d_aw_bias", "3d_aa", "bcast_aw", "2d_wa"])
def test_matmul_cpu_layer(case, dt):
    """mx.matmul (mx/matmul.py:32-200): 2-D x 2-D with a bias and the second operand in the weight format,
    batched x batched, a batched first operand against a 2-D second one, and weight x activation."""
    from microxcaling_amd.matmul import matmul
    x, w, b, a2, go, go2 = (fx("in/" + n) for n in ("x", "w", "b", "a2", "go", "go2"))
    wt = w.t().contiguous()
    m1, m2, mb, mode, mgo = {"2d_aw_bias": (x[0], wt, b, "aw", go[0]), "3d_aa": (x, a2, None, "aa", go2),
                             "bcast_aw": (x, wt, None, "aw", go),
                             "2d_wa": (w, x[1].t().contiguous(), None, "wa", go[1].t().contiguous())}[case]
    specs = _specs(w_elem_format="fp4_e2m1", a_elem_format="fp8_e4m3", block_size=32, bfloat=16,
                   quantize_backprop=True)
    i1, i2 = m1.to(DT[dt]).clone().requires_grad_(True), m2.to(DT[dt]).clone().requires_grad_(True)
    ib = None if mb is None else mb.to(DT[dt]).clone().requires_grad_(True)
    out = matmul(i1, i2, bias=ib, mx_specs=specs, mode_config=mode)
    out.backward(mgo.to(DT[dt]))
    key = "matmul/%s/%s/" % (case, dt)
    assert_bits_equal(out.detach(), fx(key + "out"), "forward")
    assert_bits_equal(i1.grad, fx(key + "g1"), "grad_in1")
    assert_bits_equal(i2.grad, fx(key + "g2"), "grad_in2")
    if ib is not None:
        assert_bits_equal(ib.grad, fx(key + "gb"), "grad_bias")


VEC_SPECS = {"bfloat16": dict(bfloat=16), "fp16": dict(fp=16),
             "exp2_recip": dict(bfloat=16, vec_use_exp2=True, vec_use_recip=True),
             "floor": dict(bfloat=16, round="floor"), "none": dict()}


@pytest.mark.parametrize("dt", ["f32", "bf16"])
@pytest.mark.parametrize("variant", list(VEC_SPECS))
def test_vector_ops_on_cpu_tensors(variant, dt):
    """The vec_* ops on their own (mx/vector_ops.py:38-128): a tensor op followed by the elementwise
    quantizer, in its bfloat16 / fp16 / round-down forms, with the 2^x and reciprocal variants, and
    with no format at all."""
    from microxcaling_amd import vector_ops as V
    from microxcaling_amd.specs import finalize_mx_specs
    sp = finalize_mx_specs(dict(VEC_SPECS[variant]), early_exit=False)
    a, b = fx("in/nx")[0].to(DT[dt]), (fx("in/ngo")[0] + 0.25).to(DT[dt])
    key = "vec/%s/%s/" % (variant, dt)
    got = {"quantize": V.vec_quantize(a, mx_specs=sp), "add": V.vec_add(a, b, mx_specs=sp),
           "sub": V.vec_sub(a, b, mx_specs=sp), "mul": V.vec_mul(a, b, mx_specs=sp),
           "div": V.vec_div(a, b, mx_specs=sp), "exp": V.vec_exp(a, mx_specs=sp),
           "exp2": V.vec_exp2(a, mx_specs=sp), "recip": V.vec_recip(b, mx_specs=sp),
           "sqrt": V.vec_sqrt(a.abs(), mx_specs=sp), "tanh": V.vec_tanh(a, mx_specs=sp),
           "reduce_sum": V.vec_reduce_sum(a, 1, keepdim=True, mx_specs=sp)}
    if not VEC_SPECS[variant].get("vec_use_recip"):
        got["reduce_mean"] = V.vec_reduce_mean(a, [0, 1], mx_specs=sp)
    for name, t in got.items():
        assert_bits_equal(t, fx(key + name), "vec_" + name)


@pytest.mark.parametrize("dt", ["f32", "bf16"])
def test_attention_scores_oracle_and_cpu_layer(dt):
    """softmax(bmm(a, b)) over the last axis (mx/bmm.py:132-138, mx/softmax.py:91-97): the oracle's chain and
    mx.bmm_softmax, which on CPU tensors -- and whenever a gradient is wanted -- is the two layers in a row."""
    a, b, go = (fx("in/" + n).to(DT[dt]) for n in ("x", "a2", "go2"))
    key = "bmm_softmax/%s/" % dt
    logits = O.mx_bmm_forward(a, b, "fp6_e2m3", bfloat=16)
    assert_bits_equal(O.softmax_forward(logits, -1, bfloat=16), fx(key + "out"), "oracle forward")

    from microxcaling_amd.bmm import bmm_softmax
    specs = _specs(a_elem_format="fp6_e2m3", block_size=32, bfloat=16, quantize_backprop=True)
    ai, bi = a.clone().requires_grad_(True), b.clone().requires_grad_(True)
    o = bmm_softmax(ai, bi, mx_specs=specs)
    o.backward(go)
    assert_bits_equal(o.detach(), fx(key + "out"), "layer forward")
    assert_bits_equal(ai.grad, fx(key + "g1"), "layer grad_in1")
    assert_bits_equal(bi.grad, fx(key + "g2"), "layer grad_in2")
    with torch.no_grad():
        assert_bits_equal(bmm_softmax(a, b, mx_specs=specs), fx(key + "out"), "layer forward, no gradient")
        plain = bmm_softmax(a, b, mx_specs=None)
    assert torch.equal(plain, torch.softmax(torch.bmm(a, b), dim=-1))


@pytest.mark.parametrize("dt", ["f32", "bf16"])
@pytest.mark.parametrize("exp2", [False, True])
def test_softmax_oracle_and_cpu_layer(dt, exp2):
    x, go = fx("in/sx").to(DT[dt]), fx("in/sgo").to(DT[dt])
    key = "softmax/%s/exp2_%d/" % (dt, int(exp2))
    out = O.softmax_forward(x, -1, bfloat=16, use_exp2=exp2)
    assert_bits_equal(out, fx(key + "out"), "oracle forward")
    assert_bits_equal(O.softmax_backward(out, go, -1, bfloat=16, use_exp2=exp2), fx(key + "gx"),
                      "oracle backward")

    from microxcaling_amd.softmax import softmax
    specs = _specs(bfloat=16, softmax_exp2=exp2, quantize_backprop=True)
    xi = x.clone().requires_grad_(True)
    o = softmax(xi, dim=-1, mx_specs=specs)
    o.backward(go)
    assert_bits_equal(o.detach(), fx(key + "out"), "layer forward")
    assert_bits_equal(xi.grad, fx(key + "gx"), "layer backward")


@pytest.mark.parametrize("dt", ["f32", "bf16"])
def test_softmax_switches(dt):
    """vec_use_exp2 (2^Q(x log2 e)), vec_use_recip (e * Q(1 / sum)) and an fp format."""
    from microxcaling_amd.softmax import softmax
    x = fx("in/sx").to(DT[dt])
    for sw in ("vec_use_exp2", "vec_use_recip"):
        want = fx("softmax/%s/%s/out" % (dt, sw))
        assert_bits_equal(O.softmax_forward(x, -1, bfloat=16, **{sw: True}), want, "oracle " + sw)
        assert_bits_equal(softmax(x, dim=-1, mx_specs=_specs(bfloat=16, **{sw: True})), want, "layer " + sw)
    want = fx("softmax/%s/fp16/out" % dt)
    assert_bits_equal(O.softmax_forward(x, -1, bfloat=0, fp=16), want, "oracle fp16")
    assert_bits_equal(softmax(x, dim=-1, mx_specs=_specs(fp=16)), want, "layer fp16")


@pytest.mark.parametrize("dt", ["f32", "bf16"])
@pytest.mark.parametrize("layer", ["layernorm", "rmsnorm"])
def test_norm_layers_on_cpu(dt, layer):
    from microxcaling_amd.layernorm import LayerNorm, RMSNorm
    specs = _specs(bfloat=16, quantize_backprop=True)
    m = {"layernorm": LayerNorm, "rmsnorm": RMSNorm}[layer](64, eps=1e-5, mx_specs=specs).to(DT[dt])
    with torch.no_grad():
        m.weight.copy_(fx("in/nw").to(DT[dt]))
        m.bias.copy_(fx("in/nb").to(DT[dt]))
    x = fx("in/nx").to(DT[dt]).clone().requires_grad_(True)
    out = m(x)
    out.backward(fx("in/ngo").to(DT[dt]))
    key = "%s/%s/" % (layer, dt)
    assert_bits_equal(out.detach(), fx(key + "out"), "forward")
    assert_bits_equal(x.grad, fx(key + "gx"), "grad_input")
    assert_bits_equal(m.weight.grad, fx(key + "gw"), "grad_weight")
    assert_bits_equal(m.bias.grad, fx(key + "gb"), "grad_bias")


@pytest.mark.parametrize("dt", ["f32", "bf16"])
@pytest.mark.parametrize("name", ["sigmoid", "tanh", "relu", "relu6", "leaky_relu", "silu", "gelu", "gelu1"])
def test_activations_on_cpu(dt, name):
    from microxcaling_amd import activations as act
    specs = _specs(bfloat=16, quantize_backprop=True)
    fn = {"sigmoid": lambda t: act.sigmoid(t, mx_specs=specs), "tanh": lambda t: act.tanh(t, mx_specs=specs),
          "relu": lambda t: act.relu(t, mx_specs=specs), "relu6": lambda t: act.relu6(t, mx_specs=specs),
          "leaky_relu": lambda t: act.leaky_relu(t, 0.1, mx_specs=specs),
          "silu": lambda t: act.silu(t, mx_specs=specs), "gelu": lambda t: act.gelu(t, mx_specs=specs),
          "gelu1": lambda t: act.gelu(t, mx_specs=specs, first_order_gelu=True)}[name]
    x = (fx("in/nx") * 2).to(DT[dt]).clone().requires_grad_(True)
    out = fn(x)
    out.backward(fx("in/ngo").to(DT[dt]))
    assert_bits_equal(out.detach(), fx("act/%s/%s/out" % (name, dt)), "forward")
    assert_bits_equal(x.grad, fx("act/%s/%s/gx" % (name, dt)), "backward")


# ---- convolutions, batch / group norm, pooling, simd ops, LSTM (fp32, bfloat16 + MXFP8 specs) ----
def _cspecs():
    return _specs(w_elem_format="fp8_e4m3", a_elem_format="fp8_e4m3", block_size=32, bfloat=16,
                  quantize_backprop=True)


def _load_params(m, key):
    with torch.no_grad():
        for n, p in m.named_parameters():
            p.copy_(fx(key + "p_" + n))


def _check_module(key, m, x, go, params=True):
    if params:
        _load_params(m, key)
    xi = x.clone().requires_grad_(True)
    out = m(xi)
    out.backward(go)
    assert_bits_equal(out.detach(), fx(key + "out"), key + "out")
    assert_bits_equal(xi.grad, fx(key + "gx"), key + "gx")
    if params:
        for n, p in m.named_parameters():
            assert_bits_equal(p.grad, fx(key + "g_" + n), key + "g_" + n)


def test_convolutions_on_cpu():
    from microxcaling_amd.convolution import Conv1d, Conv2d
    s = _cspecs()
    cx = fx("in/cx")
    _check_module("conv2d/", Conv2d(64, 48, 3, stride=2, padding=1, mx_specs=s), cx, fx("in/cgo"))
    _check_module("conv2d_groups/", Conv2d(64, 64, 3, padding=1, groups=2, bias=False, mx_specs=s), cx,
                  fx("in/cgo2"))
    _check_module("conv1d/", Conv1d(32, 40, 5, padding=2, mx_specs=s), fx("in/c1"), fx("in/c1go"))


@pytest.mark.parametrize("dt", ["f32", "bf16"])
@pytest.mark.parametrize("block", [32, 0])
@pytest.mark.parametrize("fmt", ["fp8_e4m3", "fp6_e2m3", "fp4_e2m1", "int8"])
def test_an_exponent_per_element(fmt, block, dt):
    """quantize_mx_op with shared_exp_method="none" (mx/mx_ops.py:49-92 with method "none"): every element
    takes its own exponent, whatever the block size and the axis."""
    from microxcaling_amd.mx_ops import quantize_mx_op
    specs = _specs(a_elem_format=fmt, w_elem_format=fmt, block_size=block, shared_exp_method="none")
    qa = fx("in/qa").to(DT[dt])
    for ax in (-1, 0):
        got = quantize_mx_op(qa, specs, elem_format=fmt, axes=[ax], round="nearest")
        assert_bits_equal(got, fx("mx_none/%s/block%d/%s/axis%d" % (fmt, block, dt, ax)), "axis %d" % ax)
