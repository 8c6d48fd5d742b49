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
    from microxcaling_amd.transpose_convolution import ConvTranspose2d
    s = _cspecs()
    cx = fx("in/cx")
    _check_module("conv2d/", Conv2d(64, 48, 3, stride=2, padding=1, mx_specs=s), cx, fx("in/cgo"))
    _check_module("conv2d_groups/", Conv2d(64, 64, 3, padding=1, groups=2, bias=False, mx_specs=s), cx,
                  fx("in/cgo2"))
    _check_module("conv1d/", Conv1d(32, 40, 5, padding=2, mx_specs=s), fx("in/c1"), fx("in/c1go"))
    _check_module("convT2d/", ConvTranspose2d(64, 32, 3, stride=2, padding=1, output_padding=1, mx_specs=s),
                  cx, fx("in/tgo"))


def test_batch_and_group_norm_on_cpu():
    from microxcaling_amd.batchnorm import BatchNorm2d
    from microxcaling_amd.groupnorm import GroupNorm
    s = _specs(bfloat=16, quantize_backprop=True)
    cx, go = fx("in/cx"), fx("in/bgo")
    bn = BatchNorm2d(64, mx_specs=s)
    _check_module("bn_train/", bn, cx, go)
    assert_bits_equal(bn.running_mean, fx("bn_train/running_mean"), "running_mean")
    assert_bits_equal(bn.running_var, fx("bn_train/running_var"), "running_var")
    bn.eval()
    _check_module("bn_eval/", bn, cx, go, params=False)
    _check_module("gn/", GroupNorm(4, 64, mx_specs=s), cx, go)


def test_adaptive_avg_pool_on_cpu():
    from microxcaling_amd.adaptive_avg_pooling import adaptive_avg_pool2d
    s = _specs(bfloat=16, quantize_backprop=True)
    x = fx("in/cx").clone().requires_grad_(True)
    out = adaptive_avg_pool2d(x, (2, 3), mx_specs=s)
    out.backward(fx("in/pgo"))
    assert_bits_equal(out.detach(), fx("pool/out"), "out")
    assert_bits_equal(x.grad, fx("pool/gx"), "gx")


def test_simd_ops_on_cpu():
    from microxcaling_amd import simd_ops as so
    s = _specs(bfloat=16, quantize_backprop=True)
    sa, sb, go = fx("in/sa"), fx("in/sb"), fx("in/ssgo")
    for name, fn in {"add": so.simd_add, "sub": so.simd_sub, "mul": so.simd_mul, "div": so.simd_div}.items():
        a, b = sa.clone().requires_grad_(True), sb.clone().requires_grad_(True)
        out = fn(a, b, mx_specs=s)
        out.backward(go)
        assert_bits_equal(out.detach(), fx("simd/%s/out" % name), name)
        assert_bits_equal(a.grad, fx("simd/%s/g1" % name), name + " g1")
        assert_bits_equal(b.grad, fx("simd/%s/g2" % name), name + " g2")
        a = sa.clone().requires_grad_(True)
        out = fn(a, 1.7, mx_specs=s)
        out.backward(go)
        assert_bits_equal(out.detach(), fx("simd/%s_const/out" % name), name + " const")
        assert_bits_equal(a.grad, fx("simd/%s_const/g1" % name), name + " const g1")
    for name, fn in {"square": so.simd_square, "sqrt": so.simd_sqrt, "exp": so.simd_exp, "log": so.simd_log}.items():
        a = (sa.abs() + 0.1).clone().requires_grad_(True)
        out = fn(a, mx_specs=s)
        out.backward(go)
        assert_bits_equal(out.detach(), fx("simd/%s/out" % name), name)
        assert_bits_equal(a.grad, fx("simd/%s/g1" % name), name + " g1")
    a = sa.clone().requires_grad_(True)
    out = so.simd_reduce_sum(a, [0, 2], mx_specs=s)
    out.backward(torch.ones_like(out) * 0.37)
    assert_bits_equal(out.detach(), fx("simd/reduce_sum/out"), "reduce_sum")
    assert_bits_equal(a.grad, fx("simd/reduce_sum/g1"), "reduce_sum g1")
    a = sa.clone().requires_grad_(True)
    out = so.simd_reduce_mean(a, -1, keepdim=True, mx_specs=s)
    out.backward(torch.ones_like(out) * 0.37)
    assert_bits_equal(out.detach(), fx("simd/reduce_mean/out"), "reduce_mean")
    assert_bits_equal(a.grad, fx("simd/reduce_mean/g1"), "reduce_mean g1")
    a = sa.clone().requires_grad_(True)
    out = so.simd_norm(a, mx_specs=s)
    out.backward()
    assert_bits_equal(out.detach(), fx("simd/norm/out"), "norm")
    assert_bits_equal(a.grad, fx("simd/norm/g1"), "norm g1")


def test_lstm_on_cpu():
    from torch.nn.utils.rnn import pack_padded_sequence
    from microxcaling_amd.rnn import LSTM
    m = LSTM(32, 64, num_layers=2, bidirectional=True, mx_specs=_cspecs())
    _load_params(m, "lstm/")
    x = fx("in/lx").clone().requires_grad_(True)
    out, (hn, cn) = m(x)
    (out * fx("in/lgo")).sum().backward()
    assert_bits_equal(out.detach(), fx("lstm/out"), "out")
    assert_bits_equal(hn.detach(), fx("lstm/hn"), "hn")
    assert_bits_equal(cn.detach(), fx("lstm/cn"), "cn")
    assert_bits_equal(x.grad, fx("lstm/gx"), "gx")
    for n, p in m.named_parameters():
        assert_bits_equal(p.grad, fx("lstm/g_" + n), "g_" + n)
    outp, (hn, cn) = m(pack_padded_sequence(fx("in/lx"), [5, 3, 2]))
    assert_bits_equal(outp.data.detach(), fx("lstm_packed/out"), "packed out")
    assert_bits_equal(hn.detach(), fx("lstm_packed/hn"), "packed hn")
    assert_bits_equal(cn.detach(), fx("lstm_packed/cn"), "packed cn")
