"""Writes reference_shape_sweep.json: the reference's layers on the CPU over seeded random *shapes* --
contraction lengths that are not a multiple of the block size (ragged last block along K, along the
example axis of the weight gradient, along the output axis of the input gradient), 1-D / 2-D / 4-D
inputs of linear, matmul against a 2-D and against a batched second operand, bmm, softmax over every
axis, layer norms of several widths, convolutions with stride / padding / dilation / groups in one,
two and three dimensions -- under three fixed settings.  Outputs and every gradient as SHA-256
digests (the settings sweep, gen_reference_spec_sweep.py, stores full tensors for its first cases).

Run once where the reference checkout exists:
``python tests/golden/gen_reference_shape_sweep.py /root/reference``.  Only shapes, settings and digests
of the reference's outputs are stored; none of the reference's code is."""
import hashlib
import json
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
DTYPES = {"f32": torch.float32, "bf16": torch.bfloat16}
SETTINGS = [
    dict(w_elem_format="fp8_e4m3", a_elem_format="fp8_e4m3", block_size=32, bfloat=16, custom_cuda=False),
    dict(w_elem_format="fp4_e2m1", a_elem_format="fp6_e2m3", w_elem_format_bp="fp6_e3m2", a_elem_format_bp_os="fp8_e5m2",
         block_size=16, bfloat=14, round_mx_output="even", round_grad_input="floor", custom_cuda=False),
    dict(w_elem_format="int8", a_elem_format="int4", block_size=64, scale_bits=5, fp=16, quantize_backprop=False,
         mx_flush_fp32_subnorms=True, custom_cuda=False),
]


def cases(mult=1):
    """[(kind, parameters)] -- plain lists and ints, stored in the fixture as they are.  mult: that many times
    as many cases of every kind (a longer sweep; the committed fixture is mult = 1)."""
    rng = np.random.default_rng(271828)
    r = lambda lo, hi: int(rng.integers(lo, hi + 1))
    out = []
    for _ in range(10 * mult):                                   # linear: input rank 1..4, ragged K and N
        lead = [r(1, 5) for _ in range(r(0, 3))]
        out.append(("linear", dict(lead=lead, k=r(1, 150), n=r(1, 90), bias=bool(r(0, 1)))))
    for _ in range(8 * mult):                                    # matmul: (..., m, k) x (k, n) or batched second operand
        lead = [r(1, 4) for _ in range(r(0, 2))]
        out.append(("matmul", dict(lead=lead, m=r(1, 40), k=r(1, 130), n=r(1, 70), batched2=bool(r(0, 1)) and bool(lead),
                                   bias=bool(r(0, 1)), mode=["aa", "aw", "wa"][r(0, 2)])))
    for _ in range(6 * mult):                                    # bmm
        out.append(("bmm", dict(b=r(1, 5), m=r(1, 40), k=r(1, 130), n=r(1, 70))))
    for _ in range(6 * mult):                                    # softmax over any axis
        shape = [r(1, 12) for _ in range(r(1, 4))]
        out.append(("softmax", dict(shape=shape, dim=r(-len(shape), len(shape) - 1))))
    for _ in range(6 * mult):                                    # layer norm / rms norm widths
        out.append(("norm", dict(lead=[r(1, 6) for _ in range(r(1, 2))], width=r(1, 200), rms=bool(r(0, 1)))))
    for nd in (1, 2, 3):                                  # convolutions
        for _ in range(3 * mult):
            groups = [1, 1, 2, 4][r(0, 3)]
            cin, cout = groups * r(1, 12), groups * r(1, 6)
            size = [r(5, 9) for _ in range(nd)]
            out.append(("conv", dict(nd=nd, batch=r(1, 3), cin=cin, cout=cout, size=size, k=r(1, 3), stride=r(1, 2),
                                     padding=r(0, 2), dilation=r(1, 2), groups=groups, bias=bool(r(0, 1)))))
    return out


def digest(t):
    t = t.detach().contiguous()
    f = t.float().numpy()
    raw = t.view(torch.int16 if t.element_size() == 2 else torch.int32).numpy()
    nan = np.int16(0x7FC0) if t.element_size() == 2 else np.int32(0x7FC00000)
    body = hashlib.sha256(np.ascontiguousarray(np.where(np.isnan(f), nan, raw)).tobytes()).hexdigest()
    return "%s%s:%s" % (str(t.dtype).replace("torch.", ""), list(t.shape), body)


def run_case(mx, kind, prm, setting, dt, seed):
    """One case with the layers of `mx` (the reference here, this package in the tests): {name: tensor},
    or {"raised": exception type} when the layer refuses the shape."""
    specs = mx.finalize_mx_specs(dict(setting))
    g = torch.Generator().manual_seed(seed)
    rn = lambda *s: torch.randn(*s, generator=g).to(dt)
    leaf = lambda *s: rn(*s).requires_grad_(True)
    res = {}
    try:
        if kind == "linear":
            x, w = leaf(*prm["lead"], prm["k"]), leaf(prm["n"], prm["k"])
            b = leaf(prm["n"]) if prm["bias"] else None
            o = mx.linear(x, w, b, mx_specs=specs)
            o.backward(rn(*o.shape))
            res = {"out": o, "gx": x.grad, "gw": w.grad}
            if b is not None:
                res["gb"] = b.grad
        elif kind == "matmul":
            a = leaf(*prm["lead"], prm["m"], prm["k"])
            c = leaf(*(prm["lead"] if prm["batched2"] else []), prm["k"], prm["n"])
            b = leaf(prm["n"]) if prm["bias"] else None
            o = mx.matmul(a, c, bias=b, mx_specs=specs, mode_config=prm["mode"])
            o.backward(rn(*o.shape))
            res = {"out": o, "g1": a.grad, "g2": c.grad}
            if b is not None:
                res["gb"] = b.grad
        elif kind == "bmm":
            a, c = leaf(prm["b"], prm["m"], prm["k"]), leaf(prm["b"], prm["k"], prm["n"])
            o = mx.bmm(a, c, mx_specs=specs)
            o.backward(rn(*o.shape))
            res = {"out": o, "g1": a.grad, "g2": c.grad}
        elif kind == "softmax":
            x = leaf(*prm["shape"])
            o = mx.softmax(x, dim=prm["dim"], mx_specs=specs)
            o.backward(rn(*o.shape))
            res = {"out": o, "gx": x.grad}
        elif kind == "norm":
            m = (mx.RMSNorm if prm["rms"] else mx.LayerNorm)(prm["width"], eps=1e-5, mx_specs=specs).to(dt)
            with torch.no_grad():
                m.weight.copy_(rn(prm["width"]))
                m.bias.copy_(rn(prm["width"]))
            x = leaf(*prm["lead"], prm["width"])
            o = m(x)
            o.backward(rn(*o.shape))
            res = {"out": o, "gx": x.grad, "gw": m.weight.grad, "gb": m.bias.grad}
        elif kind == "conv":
            cls = {1: mx.Conv1d, 2: mx.Conv2d, 3: mx.Conv3d}[prm["nd"]]
            m = cls(prm["cin"], prm["cout"], prm["k"], stride=prm["stride"], padding=prm["padding"],
                    dilation=prm["dilation"], groups=prm["groups"], bias=prm["bias"], mx_specs=specs)
            with torch.no_grad():
                m.weight.copy_(torch.randn(m.weight.shape, generator=g) * 0.3)
                if prm["bias"]:
                    m.bias.copy_(torch.randn(m.bias.shape, generator=g))
            m = m.to(dt)
            x = leaf(prm["batch"], prm["cin"], *prm["size"])
            o = m(x)
            o.backward(rn(*o.shape))
            res = {"out": o, "gx": x.grad, "gw": m.weight.grad}
            if prm["bias"]:
                res["gb"] = m.bias.grad
    except Exception as e:                                 # noqa: BLE001
        return {"raised": type(e).__name__}
    return res


def main(ref_root, mult=1, out_dir=HERE):
    sys.path.insert(0, ref_root)
    import mx                                            # noqa: E402
    torch.set_num_threads(1)                             # fixed summation order inside torch's CPU GEMM
    meta = {"torch": torch.__version__, "cases": [[k, p] for k, p in cases(mult)], "settings": SETTINGS, "digests": {}}
    n_raised = 0
    for ci, (kind, prm) in enumerate(cases(mult)):
        for si, setting in enumerate(SETTINGS):
            for dname, dt in DTYPES.items():
                if kind == "conv" and dname == "bf16":
                    continue
                res = run_case(mx, kind, prm, setting, dt, 1000 * ci + si)
                for k, v in res.items():
                    key = "%d/%d/%s/%s" % (ci, si, dname, k)
                    if isinstance(v, str):
                        meta["digests"][key] = v
                        n_raised += 1
                    else:
                        meta["digests"][key] = digest(v)
    with open(os.path.join(out_dir, "reference_shape_sweep.json"), "w") as f:
        json.dump(meta, f, indent=1, sort_keys=True)
    print("wrote", len(meta["digests"]), "digests,", n_raised, "raising runs")


if __name__ == "__main__":
    main(sys.argv[1] if len(sys.argv) > 1 else "/root/reference",
         int(sys.argv[2]) if len(sys.argv) > 2 else 1, sys.argv[3] if len(sys.argv) > 3 else HERE)
