"""Writes reference_layer_vectors.npz: forward outputs and gradients of the reference's MX layers
(linear, bmm, softmax, LayerNorm, RMSNorm, the activations, convolutions) on the CPU (``custom_cuda=False``), on small seeded inputs.  Run once, in a
container where the reference checkout exists:
``python tests/golden/gen_reference_layer_vectors.py /root/reference``.
Only inputs and the reference's outputs are stored; none of the reference's code is.  The fixtures
pin the order of the quantization steps inside the layers (oracle/mx_oracle.py: mx_linear_forward /
_backward, mx_bmm_forward / _backward, softmax_forward / _backward), which no literal vector of the
reference's own tests does."""
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))


def store(d, name, t):
    t = t.detach()
    if t.dtype == torch.bfloat16:
        d[name + ":bf16"] = t.contiguous().view(torch.int16).numpy().copy()
    else:
        d[name + ":f32"] = t.contiguous().view(torch.int32).numpy().copy()


def main(ref_root):
    sys.path.insert(0, ref_root)
    from mx.specs import finalize_mx_specs
    from mx.linear import linear
    from mx.bmm import bmm
    from mx.softmax import softmax

    torch.set_num_threads(1)                      # fixed summation order inside torch's CPU GEMM
    d = {}
    g = torch.Generator().manual_seed(77)
    x = torch.randn(2, 32, 64, generator=g)
    w = torch.randn(48, 64, generator=g) * 0.2
    b = torch.randn(48, generator=g)
    go = torch.randn(2, 32, 48, generator=g)
    a2 = torch.randn(2, 64, 48, generator=g)
    go2 = torch.randn(2, 32, 48, generator=g)
    sx = torch.randn(4, 128, generator=g) * 2
    sgo = torch.randn(4, 128, generator=g)
    for name, t in (("x", x), ("w", w), ("b", b), ("go", go), ("a2", a2), ("go2", go2), ("sx", sx), ("sgo", sgo)):
        store(d, "in/" + name, t)

    for dt_name, dt in (("f32", torch.float32), ("bf16", torch.bfloat16)):
        for bfloat in (0, 16):
            specs = finalize_mx_specs(dict(w_elem_format="fp8_e4m3", a_elem_format="fp8_e4m3", block_size=32,
                                           bfloat=bfloat, quantize_backprop=True, custom_cuda=False))
            xi, wi, bi = (t.to(dt).clone().requires_grad_(True) for t in (x, w, b))
            out = linear(xi, wi, bi, mx_specs=specs)
            out.backward(go.to(dt))
            key = "linear/%s/bfloat%d/" % (dt_name, bfloat)
            store(d, key + "out", out)
            store(d, key + "gx", xi.grad)
            store(d, key + "gw", wi.grad)
            store(d, key + "gb", bi.grad)

        specs = finalize_mx_specs(dict(a_elem_format="fp6_e2m3", block_size=32, quantize_backprop=True,
                                       custom_cuda=False))
        ai, bi2 = x.to(dt).clone().requires_grad_(True), a2.to(dt).clone().requires_grad_(True)
        out = bmm(ai, bi2, mx_specs=specs)
        out.backward(go2.to(dt))
        key = "bmm/%s/" % dt_name
        store(d, key + "out", out)
        store(d, key + "g1", ai.grad)
        store(d, key + "g2", bi2.grad)

        for exp2 in (False, True):
            specs = finalize_mx_specs(dict(bfloat=16, softmax_exp2=exp2, quantize_backprop=True,
                                           custom_cuda=False))
            si = sx.to(dt).clone().requires_grad_(True)
            out = softmax(si, dim=-1, mx_specs=specs)
            out.backward(sgo.to(dt))
            key = "softmax/%s/exp2_%d/" % (dt_name, int(exp2))
            store(d, key + "out", out)
            store(d, key + "gx", si.grad)
        for sw in ("vec_use_exp2", "vec_use_recip"):
            specs = finalize_mx_specs({"bfloat": 16, sw: True, "quantize_backprop": True, "custom_cuda": False})
            store(d, "softmax/%s/%s/out" % (dt_name, sw), softmax(sx.to(dt), dim=-1, mx_specs=specs))
        specs = finalize_mx_specs(dict(fp=16, quantize_backprop=True, custom_cuda=False))
        store(d, "softmax/%s/fp16/out" % dt_name, softmax(sx.to(dt), dim=-1, mx_specs=specs))

    # normalization layers and activations (bfloat16 vector-op chains)
    from mx.layernorm import LayerNorm, RMSNorm
    from mx import activations as act
    nx = torch.randn(2, 16, 64, generator=g) * 2 + 0.5
    nw = torch.randn(64, generator=g)
    nb = torch.randn(64, generator=g)
    ngo = torch.randn(2, 16, 64, generator=g)
    for name, t in (("nx", nx), ("nw", nw), ("nb", nb), ("ngo", ngo)):
        store(d, "in/" + name, t)
    specs = finalize_mx_specs(dict(bfloat=16, quantize_backprop=True, custom_cuda=False))
    for dt_name, dt in (("f32", torch.float32), ("bf16", torch.bfloat16)):
        for lname, cls in (("layernorm", LayerNorm), ("rmsnorm", RMSNorm)):
            m = cls(64, eps=1e-5, mx_specs=specs).to(dt)
            with torch.no_grad():
                m.weight.copy_(nw.to(dt))
                m.bias.copy_(nb.to(dt))
            xi = nx.to(dt).clone().requires_grad_(True)
            out = m(xi)
            out.backward(ngo.to(dt))
            key = "%s/%s/" % (lname, dt_name)
            store(d, key + "out", out)
            store(d, key + "gx", xi.grad)
            store(d, key + "gw", m.weight.grad)
            store(d, key + "gb", m.bias.grad)
        acts = {"sigmoid": lambda t: act.sigmoid(t, mx_specs=specs), "tanh": lambda t: act.tanh(t, mx_specs=specs),
                "relu": lambda t: act.relu(t, mx_specs=specs), "relu6": lambda t: act.relu6(t, mx_specs=specs),
                "leaky_relu": lambda t: act.leaky_relu(t, 0.1, mx_specs=specs),
                "silu": lambda t: act.silu(t, mx_specs=specs), "gelu": lambda t: act.gelu(t, mx_specs=specs),
                "gelu1": lambda t: act.gelu(t, mx_specs=specs, first_order_gelu=True)}
        for aname, fn in acts.items():
            xi = (nx * 2).to(dt).clone().requires_grad_(True)
            out = fn(xi)
            out.backward(ngo.to(dt))
            store(d, "act/%s/%s/out" % (aname, dt_name), out)
            store(d, "act/%s/%s/gx" % (aname, dt_name), xi.grad)

    # convolutions (fp32 tensors)
    from mx.convolution import Conv1d, Conv2d
    cspecs = finalize_mx_specs(dict(w_elem_format="fp8_e4m3", a_elem_format="fp8_e4m3", block_size=32,
                                    bfloat=16, quantize_backprop=True, custom_cuda=False))

    def run_module(key, m, x, go, params=True):
        xi = x.clone().requires_grad_(True)
        out = m(xi)
        out.backward(go)
        store(d, key + "out", out)
        store(d, key + "gx", xi.grad)
        if params:
            for n, p in m.named_parameters():
                store(d, key + "g_" + n, p.grad)
                store(d, key + "p_" + n, p)

    cx = torch.randn(2, 64, 9, 9, generator=g)
    store(d, "in/cx", cx)
    torch.manual_seed(11)
    m = Conv2d(64, 48, 3, stride=2, padding=1, mx_specs=cspecs)
    o = m(cx)
    cgo = torch.randn(o.shape, generator=g)
    store(d, "in/cgo", cgo)
    run_module("conv2d/", m, cx, cgo)
    m = Conv2d(64, 64, 3, padding=1, groups=2, bias=False, mx_specs=cspecs)
    cgo2 = torch.randn(m(cx).shape, generator=g)
    store(d, "in/cgo2", cgo2)
    run_module("conv2d_groups/", m, cx, cgo2)
    c1 = torch.randn(3, 32, 20, generator=g)
    store(d, "in/c1", c1)
    m = Conv1d(32, 40, 5, padding=2, mx_specs=cspecs)
    c1go = torch.randn(m(c1).shape, generator=g)
    store(d, "in/c1go", c1go)
    run_module("conv1d/", m, c1, c1go)

    # linear layers whose blocks do not divide the example axis of a 3-D input (block sizes 64 and
    # "whole axis"): the weight gradient shares exponents per batch entry (mx/linear.py:124-143)
    x3 = torch.randn(3, 96, 64, generator=g)
    go3 = torch.randn(3, 96, 48, generator=g)
    store(d, "in/x3", x3)
    store(d, "in/go3", go3)
    for block in (64, 0):
        bspecs = finalize_mx_specs(dict(w_elem_format="fp8_e4m3", a_elem_format="fp8_e4m3", block_size=block,
                                        bfloat=16, quantize_backprop=True, custom_cuda=False))
        xi, wi, bi = (t.clone().requires_grad_(True) for t in (x3, w, b))
        out = linear(xi, wi, bi, mx_specs=bspecs)
        out.backward(go3)
        key = "linear_block%d/" % block
        store(d, key + "out", out)
        store(d, key + "gx", xi.grad)
        store(d, key + "gw", wi.grad)
        store(d, key + "gb", bi.grad)

    # a layer with prequantized weights (mx/linear.py:246-274): weight and bias stored as bf16 once,
    # inference on bf16 and on fp32 inputs (the bf16 weight then meets an input of another dtype, 77-80)
    from mx.linear import Linear
    pspecs = finalize_mx_specs(dict(w_elem_format="fp8_e4m3", a_elem_format="fp8_e4m3", block_size=32,
                                    bfloat=16, round="even", custom_cuda=False))
    m = Linear(64, 48, bias=True, mx_specs=pspecs)
    with torch.no_grad():
        m.weight.copy_(w)
        m.bias.copy_(b)
    m.prequantize_weights()
    m.eval()
    store(d, "linear_prequantized/p_weight", m.weight.data)
    store(d, "linear_prequantized/p_bias", m.bias.data)
    with torch.no_grad():
        store(d, "linear_prequantized/out_bf16", m(x.to(torch.bfloat16)))
        store(d, "linear_prequantized/out_f32", m(x))

    # attention scores: softmax over the last axis of a batched product (mx/bmm.py:132-138 followed by
    # mx/softmax.py:91-97), forward and the gradients of both operands
    aspecs = finalize_mx_specs(dict(a_elem_format="fp6_e2m3", block_size=32, bfloat=16, quantize_backprop=True,
                                    custom_cuda=False))
    for dt_name, dt in (("f32", torch.float32), ("bf16", torch.bfloat16)):
        ai, bi2 = x.to(dt).clone().requires_grad_(True), a2.to(dt).clone().requires_grad_(True)
        out = softmax(bmm(ai, bi2, mx_specs=aspecs), dim=-1, mx_specs=aspecs)
        out.backward(go2.to(dt))
        key = "bmm_softmax/%s/" % dt_name
        store(d, key + "out", out)
        store(d, key + "g1", ai.grad)
        store(d, key + "g2", bi2.grad)

    # mx.matmul (mx/matmul.py): 2-D x 2-D with a bias and the second operand in the weight format,
    # batched x batched, and a batched first operand against a 2-D second one (broadcast)
    from mx.matmul import matmul
    mspecs = finalize_mx_specs(dict(w_elem_format="fp4_e2m1", a_elem_format="fp8_e4m3", block_size=32, bfloat=16,
                                    quantize_backprop=True, custom_cuda=False))
    wt = w.t().contiguous()
    mcases = {"2d_aw_bias": (x[0], wt, b, "aw", go[0]), "3d_aa": (x, a2, None, "aa", go2),
              "bcast_aw": (x, wt, None, "aw", go), "2d_wa": (w, x[1].t().contiguous(), None, "wa", go[1].t().contiguous())}
    for cname, (m1, m2, mb, mode, mgo) in mcases.items():
        for dt_name, dt in (("f32", torch.float32), ("bf16", torch.bfloat16)):
            i1, i2 = m1.to(dt).clone().requires_grad_(True), m2.to(dt).clone().requires_grad_(True)
            ib = None if mb is None else mb.to(dt).clone().requires_grad_(True)
            out = matmul(i1, i2, bias=ib, mx_specs=mspecs, mode_config=mode)
            out.backward(mgo.to(dt))
            key = "matmul/%s/%s/" % (cname, dt_name)
            store(d, key + "out", out)
            store(d, key + "g1", i1.grad)
            store(d, key + "g2", i2.grad)
            if ib is not None:
                store(d, key + "gb", ib.grad)

    # the vector ops (mx/vector_ops.py:38-128) on their own: bfloat16, fp16 format, the exp2 / reciprocal
    # variants, and no format at all; fp32 and bf16 tensors
    from mx import vector_ops as V
    va = nx[0]
    vb = ngo[0] + 0.25
    vspecs = {"bfloat16": dict(bfloat=16), "fp16": dict(fp=16), "exp2_recip": dict(bfloat=16, vec_use_exp2=True,
              vec_use_recip=True), "floor": dict(bfloat=16, round="floor"), "none": dict()}
    for vname, kw in vspecs.items():
        sp = finalize_mx_specs(dict(custom_cuda=False, **kw), early_exit=False)
        for dt_name, dt in (("f32", torch.float32), ("bf16", torch.bfloat16)):
            a_, b_ = va.to(dt), vb.to(dt)
            key = "vec/%s/%s/" % (vname, dt_name)
            store(d, key + "quantize", V.vec_quantize(a_, mx_specs=sp))
            store(d, key + "add", V.vec_add(a_, b_, mx_specs=sp))
            store(d, key + "sub", V.vec_sub(a_, b_, mx_specs=sp))
            store(d, key + "mul", V.vec_mul(a_, b_, mx_specs=sp))
            store(d, key + "div", V.vec_div(a_, b_, mx_specs=sp))
            store(d, key + "exp", V.vec_exp(a_, mx_specs=sp))
            store(d, key + "exp2", V.vec_exp2(a_, mx_specs=sp))
            store(d, key + "recip", V.vec_recip(b_, mx_specs=sp))
            store(d, key + "sqrt", V.vec_sqrt(a_.abs(), mx_specs=sp))
            store(d, key + "tanh", V.vec_tanh(a_, mx_specs=sp))
            store(d, key + "reduce_sum", V.vec_reduce_sum(a_, 1, keepdim=True, mx_specs=sp))
            if not kw.get("vec_use_recip"):       # the reference hands a numpy scalar to the quantizer there
                store(d, key + "reduce_mean", V.vec_reduce_mean(a_, [0, 1], mx_specs=sp))

    # quantize_mx_op with shared_exp_method="none" (an exponent per element, mx/mx_ops.py:49-92 with
    # method "none"), along the last and along the first axis, with and without blocks
    from mx.mx_ops import quantize_mx_op
    qa = nx[0] * torch.exp2(torch.randint(-6, 7, nx[0].shape, generator=g).float())
    store(d, "in/qa", qa)
    for fmt in ("fp8_e4m3", "fp6_e2m3", "fp4_e2m1", "int8"):
        for block in (32, 0):
            nspecs = finalize_mx_specs(dict(a_elem_format=fmt, w_elem_format=fmt, block_size=block,
                                            shared_exp_method="none", custom_cuda=False))
            for dt_name, dt in (("f32", torch.float32), ("bf16", torch.bfloat16)):
                for ax in (-1, 0):
                    store(d, "mx_none/%s/block%d/%s/axis%d" % (fmt, block, dt_name, ax),
                          quantize_mx_op(qa.to(dt), nspecs, elem_format=fmt, axes=[ax], round="nearest"))

    np.savez_compressed(os.path.join(HERE, "reference_layer_vectors.npz"), **d)
    print("wrote %d arrays, torch %s" % (len(d), torch.__version__))


if __name__ == "__main__":
    main(sys.argv[1] if len(sys.argv) > 1 else "/root/reference")
