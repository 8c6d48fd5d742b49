"""Writes reference_fp16_layer_vectors.npz: forward outputs and gradients of the reference's layers on
float16 *tensors* (CPU, ``custom_cuda=False``), where every quantization step runs in fp16
(mx/elemwise_ops.py:127-163, mx/mx_ops.py:265-292).  Run once, in a container where the reference
checkout exists:  ``python tests/golden/gen_reference_fp16_layer_vectors.py /root/reference``.
Only inputs and the reference's outputs are stored; none of the reference's code is."""
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
# (name, spec entries): an MX format with the bfloat16 vector format, and with the fp16 vector format
SPEC_CASES = [("mxfp8_bfloat16", dict(w_elem_format="fp8_e4m3", a_elem_format="fp8_e4m3", block_size=32, bfloat=16)),
              ("mxfp6_fp16", dict(w_elem_format="fp6_e2m3", a_elem_format="fp6_e2m3", block_size=32, fp=16)),
              ("mxfp4_floor", dict(w_elem_format="fp4_e2m1", a_elem_format="fp4_e2m1", block_size=32, bfloat=16,
                                   round="floor"))]


def inputs():
    g = torch.Generator().manual_seed(1601)
    t = {"x": torch.randn(2, 32, 64, generator=g), "w": torch.randn(48, 64, generator=g) * 0.2,
         "b": torch.randn(48, generator=g), "go": torch.randn(2, 32, 48, generator=g),
         "a2": torch.randn(2, 64, 48, generator=g), "sx": torch.randn(4, 128, generator=g) * 2,
         "sgo": torch.randn(4, 128, generator=g), "nx": torch.randn(2, 16, 64, generator=g) * 2 + 0.5,
         "nw": torch.randn(64, generator=g), "nb": torch.randn(64, generator=g),
         "ngo": torch.randn(2, 16, 64, generator=g)}
    return {k: v.to(torch.float16) for k, v in t.items()}


def main(ref_root):
    sys.path.insert(0, ref_root)
    from mx.specs import finalize_mx_specs
    from mx.linear import linear
    from mx.bmm import bmm
    from mx.softmax import softmax
    from mx.layernorm import LayerNorm, RMSNorm

    torch.set_num_threads(1)                      # fixed summation order inside torch's CPU GEMM
    t = inputs()
    d = {}

    def store(name, v):
        assert v.dtype == torch.float16, (name, v.dtype)
        d[name] = v.detach().contiguous().view(torch.int16).numpy().copy()

    for name, entries in SPEC_CASES:
        specs = finalize_mx_specs(dict(entries, quantize_backprop=True, custom_cuda=False))
        xi, wi, bi = (t[k].clone().requires_grad_(True) for k in ("x", "w", "b"))
        out = linear(xi, wi, bi, mx_specs=specs)
        out.backward(t["go"])
        for k, v in (("out", out), ("gx", xi.grad), ("gw", wi.grad), ("gb", bi.grad)):
            store("linear/%s/%s" % (name, k), v)
        ai, bi2 = t["x"].clone().requires_grad_(True), t["a2"].clone().requires_grad_(True)
        out = bmm(ai, bi2, mx_specs=specs)
        out.backward(t["go"])
        for k, v in (("out", out), ("g1", ai.grad), ("g2", bi2.grad)):
            store("bmm/%s/%s" % (name, k), v)
        si = t["sx"].clone().requires_grad_(True)
        out = softmax(si, dim=-1, mx_specs=specs)
        out.backward(t["sgo"])
        store("softmax/%s/out" % name, out)
        store("softmax/%s/gx" % name, si.grad)
        for lname, cls in (("layernorm", LayerNorm), ("rmsnorm", RMSNorm)):
            m = cls(64, eps=1e-5, mx_specs=specs).to(torch.float16)
            with torch.no_grad():
                m.weight.copy_(t["nw"])
                m.bias.copy_(t["nb"])
            xi = t["nx"].clone().requires_grad_(True)
            out = m(xi)
            out.backward(t["ngo"])
            for k, v in (("out", out), ("gx", xi.grad), ("gw", m.weight.grad), ("gb", m.bias.grad)):
                store("%s/%s/%s" % (lname, name, k), v)
    np.savez_compressed(os.path.join(HERE, "reference_fp16_layer_vectors.npz"), **d)
    print("wrote %d arrays" % len(d))


if __name__ == "__main__":
    main(sys.argv[1] if len(sys.argv) > 1 else "/root/reference")
