"""Writes reference_spec_sweep.json (+ .npz): the reference's layers on the CPU under 40 seeded random
``mx_specs`` in which every role has its own setting -- weight / activation formats for forward and
for each gradient (mx/specs.py:84-91), every ``round_*`` key (mx/specs.py:104-116), bfloat / fp
widths, bfloat_subnorms, quantize_backprop, block size, scale bits, flush, softmax_exp2 /
vec_use_exp2 / vec_use_recip -- so that a layer applying the wrong role's format or rounding
anywhere in forward or backward produces other bits.  Per case: linear, matmul (+bias), bmm, softmax,
LayerNorm, RMSNorm, seven activations, quantize_bfloat, Conv2d -- outputs and every gradient, fp32 and
bf16 tensors, as
SHA-256 digests; the first four cases are also stored in full.

Run once where the reference checkout exists:
``python tests/golden/gen_reference_spec_sweep.py /root/reference``.  Only inputs, settings and the
reference's outputs are stored; none of the reference's code is."""
import hashlib
import json
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
FORMATS = ["fp8_e4m3", "fp8_e5m2", "fp6_e3m2", "fp6_e2m3", "fp4_e2m1", "int8", "int4"]
ROUNDS = ["nearest", "floor", "even"]
ROUND_KEYS = ["round", "round_m", "round_weight", "round_output", "round_grad_weight", "round_grad_input",
              "round_mx_output", "round_mx_input_grad_input", "round_mx_weight_grad_input",
              "round_mx_grad_output_grad_input", "round_mx_input_grad_weight", "round_mx_grad_output_grad_weight"]
N_CASES = 40
N_STORED = 4
DTYPES = {"f32": torch.float32, "bf16": torch.bfloat16}


def spec_cases(n_cases=N_CASES):
    """The sweep's settings (plain dicts, before finalize_mx_specs)."""
    rng = np.random.default_rng(314159)
    pick = lambda seq: seq[int(rng.integers(len(seq)))]
    cases = []
    for i in range(n_cases):
        d = {"custom_cuda": False}
        d["w_elem_format"] = pick(FORMATS)
        d["a_elem_format"] = pick(FORMATS)
        for k in ("w_elem_format_bp", "a_elem_format_bp", "a_elem_format_bp_ex", "a_elem_format_bp_os"):
            if rng.integers(3):
                d[k] = pick(FORMATS)
        if i % 10 == 9:                       # one role left unquantized
            d[pick(["w_elem_format", "a_elem_format"])] = None
        d["block_size"] = pick([32, 32, 16, 64, 8])
        d["scale_bits"] = pick([8, 8, 5])
        width = pick([16, 16, 14, 12, 0])
        if rng.integers(4) == 0 and width:
            d["fp"] = pick([16, 14, 12])
        else:
            d["bfloat"] = width
        d["bfloat_subnorms"] = bool(rng.integers(4))
        d["quantize_backprop"] = bool(rng.integers(4))
        d["mx_flush_fp32_subnorms"] = bool(rng.integers(2))
        for k in ROUND_KEYS:
            d[k] = pick(ROUNDS)
        if d.get("bfloat") == 16:
            # round 'even' at 16 bits is a dtype cast in the reference (mx/elemwise_ops.py:248-251): fp32
            # tensors would turn into bf16 ones mid-layer; keep the elementwise roundings off that shortcut
            for k in ("round", "round_weight", "round_output", "round_grad_weight", "round_grad_input"):
                if d[k] == "even":
                    d[k] = "floor"
        d["softmax_exp2"] = bool(rng.integers(2))
        d["vec_use_exp2"] = bool(rng.integers(3) == 0)
        d["vec_use_recip"] = bool(rng.integers(3) == 0)
        cases.append(d)
    return cases


def inputs():
    g = torch.Generator().manual_seed(2718)
    r = lambda *s: torch.randn(*s, generator=g)
    return {
        "x": r(3, 20, 64), "w": r(40, 64) * 0.3, "b": r(40), "go": r(3, 20, 40),
        "m1": r(24, 64), "m2": r(64, 40) * 0.3, "mgo": r(24, 40),
        "a": r(2, 24, 64), "c": r(2, 64, 40), "bgo": r(2, 24, 40),
        "sx": r(5, 96) * 2, "sgo": r(5, 96),
        "nx": r(6, 64) * 2 + 0.5, "nw": r(64), "nb": r(64), "ngo": r(6, 64),
        "cx": r(2, 32, 7, 7), "cw": r(16, 32, 3, 3) * 0.2, "cb": r(16), "cgo": r(2, 16, 7, 7),
    }


def bits_of(t):
    return t.detach().contiguous().view(torch.int16 if t.element_size() == 2 else torch.int32).numpy().copy()


def digest(t):
    t = t.detach().contiguous()
    f = t.float().numpy()
    if t.element_size() == 2:
        b = np.where(np.isnan(f), np.int16(0x7FC0), bits_of(t))
    else:
        b = np.where(np.isnan(f), np.int32(0x7FC00000), bits_of(t))
    return "%s:%s" % (str(t.dtype).replace("torch.", ""), hashlib.sha256(np.ascontiguousarray(b).tobytes()).hexdigest())


def run_case(mx, raw, inp, dt):
    """Every layer of the sweep under one setting: {name: tensor}.  `mx` is the package under test (the
    reference here; the tests pass this package's modules)."""
    specs = mx.finalize_mx_specs(dict(raw))
    T = {k: v.to(dt) for k, v in inp.items()}
    leaf = lambda k: T[k].clone().requires_grad_(True)
    out = {}

    def ran(name, fn):
        try:
            fn()
        except Exception as e:                              # noqa: BLE001
            out[name + "/raised"] = type(e).__name__

    def linear_():
        x, w, b = leaf("x"), leaf("w"), leaf("b")
        o = mx.linear(x, w, b, mx_specs=specs)
        o.backward(T["go"])
        out.update({"linear/out": o, "linear/gx": x.grad, "linear/gw": w.grad, "linear/gb": b.grad})

    def matmul_():
        m1, m2, b = leaf("m1"), leaf("m2"), leaf("b")
        o = mx.matmul(m1, m2, bias=b, mx_specs=specs)
        o.backward(T["mgo"])
        out.update({"matmul/out": o, "matmul/g1": m1.grad, "matmul/g2": m2.grad, "matmul/gb": b.grad})

    def bmm_():
        a, c = leaf("a"), leaf("c")
        o = mx.bmm(a, c, mx_specs=specs)
        o.backward(T["bgo"])
        out.update({"bmm/out": o, "bmm/g1": a.grad, "bmm/g2": c.grad})

    def softmax_():
        s = leaf("sx")
        o = mx.softmax(s, dim=-1, mx_specs=specs)
        o.backward(T["sgo"])
        out.update({"softmax/out": o, "softmax/gx": s.grad})

    def norm_(name, cls):
        def f():
            m = cls(64, eps=1e-5, mx_specs=specs).to(dt)
            with torch.no_grad():
                m.weight.copy_(T["nw"])
                m.bias.copy_(T["nb"])
            x = leaf("nx")
            o = m(x)
            o.backward(T["ngo"])
            out.update({name + "/out": o, name + "/gx": x.grad, name + "/gw": m.weight.grad, name + "/gb": m.bias.grad})
        return f

    def act_(name, fn):
        def f():
            x = leaf("nx")
            o = fn(x, mx_specs=specs)
            o.backward(T["ngo"])
            out.update({name + "/out": o, name + "/gx": x.grad})
        return f

    def conv_():
        m = mx.Conv2d(32, 16, 3, padding=1, mx_specs=specs).to(dt)
        with torch.no_grad():
            m.weight.copy_(T["cw"])
            m.bias.copy_(T["cb"])
        x = leaf("cx")
        o = m(x)
        o.backward(T["cgo"])
        out.update({"conv2d/out": o, "conv2d/gx": x.grad, "conv2d/gw": m.weight.grad, "conv2d/gb": m.bias.grad})

    ran("linear", linear_)
    ran("matmul", matmul_)
    ran("bmm", bmm_)
    ran("softmax", softmax_)
    ran("layernorm", norm_("layernorm", mx.LayerNorm))
    ran("rmsnorm", norm_("rmsnorm", mx.RMSNorm))
    ran("gelu", act_("gelu", mx.gelu))
    ran("sigmoid", act_("sigmoid", mx.sigmoid))
    ran("tanh", act_("tanh", mx.tanh))
    ran("silu", act_("silu", mx.silu))
    ran("relu6", act_("relu6", mx.relu6))
    ran("leaky_relu", act_("leaky_relu", lambda x, mx_specs: mx.leaky_relu(x, 0.05, mx_specs=mx_specs)))
    ran("gelu1", act_("gelu1", lambda x, mx_specs: mx.gelu(x, mx_specs=mx_specs, first_order_gelu=True)))
    ran("quantize_bfloat", act_("quantize_bfloat", lambda x, mx_specs: mx.quantize_bfloat(x, mx_specs)))
    if dt == torch.float32:
        ran("conv2d", conv_)
    return out


def main(ref_root, n_cases=N_CASES, out_dir=HERE):
    """n_cases / out_dir other than the defaults: a longer sweep written somewhere else (digests only are
    compared by whoever reads it; the committed fixture is the default run)."""
    sys.path.insert(0, ref_root)
    import mx                                            # noqa: E402
    torch.set_num_threads(1)                             # fixed summation order inside torch's CPU GEMM
    inp = inputs()
    arrays = {"in/" + k: bits_of(v) for k, v in inp.items()}
    meta = {"torch": torch.__version__, "cases": spec_cases(n_cases), "digests": {}}
    n_raised = 0
    for i, raw in enumerate(meta["cases"]):
        for dname, dt in DTYPES.items():
            res = run_case(mx, raw, inp, dt)
            for k, v in res.items():
                key = "%d/%s/%s" % (i, dname, k)
                if isinstance(v, str):
                    meta["digests"][key] = "raised:" + v
                    n_raised += 1
                    continue
                meta["digests"][key] = digest(v)
                if i < N_STORED:
                    arrays[key] = bits_of(v)
    np.savez_compressed(os.path.join(out_dir, "reference_spec_sweep.npz"), **arrays)
    with open(os.path.join(out_dir, "reference_spec_sweep.json"), "w") as f:
        json.dump(meta, f, indent=1, sort_keys=True)
    print("wrote", len(meta["digests"]), "digests,", n_raised, "raising layer runs,", len(arrays), "arrays")


if __name__ == "__main__":
    main(sys.argv[1] if len(sys.argv) > 1 else "/root/reference",
         int(sys.argv[2]) if len(sys.argv) > 2 else N_CASES, sys.argv[3] if len(sys.argv) > 3 else HERE)
