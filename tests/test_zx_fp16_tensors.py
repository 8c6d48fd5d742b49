"""fp16 tensors.  The reference's pure path evaluates every op in fp16 on them (mx/mx_ops.py:265-292,
mx/elemwise_ops.py:127-163); tests/golden/gen_reference_fp16_vectors.py stored what it returns.  The
same bodies run against both oracles, the host library on CPU tensors and (marked gpu) the HIP kernels
through the C ABI."""
import hashlib

import numpy as np
import pytest
import torch

from helpers import GOLDEN, PackageImpl, assert_bits_equal, canon_bits, from_bits
from oracle import c_oracle as C
from oracle import mx_oracle as O

ROUNDS = ["nearest", "floor", "even"]
MX_FORMATS = ["fp8_e4m3", "fp8_e5m2", "fp6_e3m2", "fp6_e2m3", "fp4_e2m1", "int8", "int4"]
ORACLES = [pytest.param(O, id="torch"), pytest.param(C, id="c"),
           pytest.param(PackageImpl("cpu"), id="host_library"),
           pytest.param(PackageImpl("cuda"), id="hip", marks=pytest.mark.gpu)]


def _digest(t):
    return hashlib.sha256(np.ascontiguousarray(canon_bits(t)).tobytes()).hexdigest()


_fp16_golden = None


def fp16_golden():
    global _fp16_golden
    if _fp16_golden is None:
        import importlib.util
        import json
        import os
        spec = importlib.util.spec_from_file_location("gen_reference_fp16_vectors",
                                                      os.path.join(GOLDEN, "gen_reference_fp16_vectors.py"))
        mod = importlib.util.module_from_spec(spec)
        spec.loader.exec_module(mod)
        with open(os.path.join(GOLDEN, "reference_fp16_vectors.json")) as f:
            meta = json.load(f)
        _fp16_golden = (np.load(os.path.join(GOLDEN, "reference_fp16_vectors.npz")), meta, mod)
    return _fp16_golden


@pytest.mark.parametrize("orc", ORACLES)
def test_golden_fp16_mx_blocks(orc):
    """Blocks with maxima at every fp16 exponent, inside and beside the round-up zones of log2, with
    scales that overflow and underflow in fp16, zeros, Inf and NaN: the reference's outputs, stored."""
    z, _, _ = fp16_golden()
    x = from_bits(z["mx_x"], torch.float16)
    for fmt in MX_FORMATS:
        for rnd in ROUNDS:
            y = orc.quantize_mx(x.clone(), 8, fmt, axes=[-1], block_size=32, round=rnd)
            assert_bits_equal(y, from_bits(z["mx_y.%s.%s" % (fmt, rnd)], torch.float16), fmt + rnd)
    y = orc.quantize_mx(x.t().contiguous(), 5, "fp8_e4m3", axes=[0], block_size=32, round="even",
                        flush_fp32_subnorms=True)
    assert_bits_equal(y, from_bits(z["mx_y.t.fp8_e4m3.even.sb5.flush"], torch.float16), "transposed")
    y = orc.quantize_mx(x.clone(), 8, "fp6_e2m3", axes=[-1], block_size=32, round="nearest", flush_fp32_subnorms=True)
    assert_bits_equal(y, from_bits(z["mx_y.fp6_e2m3.nearest.flush"], torch.float16), "flush")
    y = orc.quantize_mx(x.clone(), 4, "int8", axes=[-1], block_size=8, round="floor")
    assert_bits_equal(y, from_bits(z["mx_y.int8.floor.sb4.bs8"], torch.float16), "scale_bits 4, blocks of 8")
    y = orc.quantize_mx(x[:, :24].contiguous(), 8, "fp4_e2m1", axes=[-1], block_size=16, round="even")
    assert_bits_equal(y, from_bits(z["mx_y.fp4_e2m1.even.ragged24.bs16"], torch.float16), "ragged last block")


@pytest.mark.parametrize("orc", ORACLES)
def test_golden_fp16_mx_every_code(orc):
    """Every finite fp16 code as an element under 14 block maxima x 7 formats x 3 roundings x scale_bits
    8 and 5: digests of the reference's outputs, two cases stored in full."""
    z, meta, gen = fp16_golden()
    n = 0
    for (exp, frac) in gen.EXHAUSTIVE_MAXIMA:
        blk = gen.exhaustive_block(exp, frac)
        for fmt in MX_FORMATS:
            for rnd in ROUNDS:
                for sb in (8, 5):
                    y = orc.quantize_mx(blk.clone(), sb, fmt, axes=[-1], block_size=32, round=rnd)
                    key = "%d.%d.%s.%s.%d" % (exp, frac, fmt, rnd, sb)
                    stored = "mx_exh_y." + key
                    if stored in z.files:
                        assert_bits_equal(y, from_bits(z[stored], torch.float16), key)
                    assert _digest(y) == meta["mx_digests"][key], key
                    n += 1
    assert n == len(meta["mx_digests"]) == 588


@pytest.mark.parametrize("orc", ORACLES)
def test_golden_fp16_elementwise_every_code(orc):
    """The elementwise quantizer on all 65 536 fp16 codes: 7 formats (bfloat16, fp16, two fp8, a 20-bit
    format whose scaled values overflow fp16, one with 6 exponent bits, int8) x 3 roundings x saturate x
    denorm.  Where the clamp bound does not fit fp16 the reference raises; so must every implementation."""
    z, meta, gen = fp16_golden()
    codes = gen.all_fp16_codes()
    n = 0
    for name, (bits, ebits, mx) in gen.ELEM_CFG.items():
        for rnd in ROUNDS:
            for sat in (False, True):
                for den in (True, False):
                    key = "%s.%s.%d.%d" % (name, rnd, sat, den)
                    if key in meta["elem_raises"]:
                        with pytest.raises(RuntimeError):
                            orc.quantize_elemwise_core(codes.clone(), bits, ebits, mx, round=rnd,
                                                       saturate_normals=sat, allow_denorm=den)
                        continue
                    y = orc.quantize_elemwise_core(codes.clone(), bits, ebits, mx, round=rnd,
                                                   saturate_normals=sat, allow_denorm=den)
                    if "elem_y." + key in z.files:
                        assert_bits_equal(y, from_bits(z["elem_y." + key], torch.float16), key)
                    assert _digest(y) == meta["elem_digests"][key], key
                    n += 1
    assert n == len(meta["elem_digests"]) == 78 and len(meta["elem_raises"]) == 6


@pytest.mark.gpu
def test_fp16_tensors_on_the_gpu():
    """Default mode: the all-fp16 arithmetic of the pure path (bit for bit against the oracle; the
    reference's own outputs are compared in test_oracle_pins.py).  Exact exponents: the widened fp32
    computation rounded back, as on CPU tensors -- bit for bit, the sign of a zero included."""
    from microxcaling_amd import custom_extensions as ce
    from microxcaling_amd.elemwise_ops import _quantize_elemwise_core
    from microxcaling_amd.mx_ops import _quantize_mx
    assert torch.cuda.is_available(), "this test needs a GPU"
    dev = torch.device("cuda:0")

    def mx_gpu(x, *a, **k):
        y = _quantize_mx(x, *a, **k)
        torch.cuda.synchronize()
        return y

    def elem_gpu(x, *a, **k):
        y = _quantize_elemwise_core(x, *a, **k)
        torch.cuda.synchronize()
        return y

    g = torch.Generator().manual_seed(2)
    x = (torch.randn(64, 256, generator=g) * 3).half()
    for axis in (-1, 0):
        for rnd in ("nearest", "floor", "even"):
            got = mx_gpu(x.to(dev), 8, "fp8_e4m3", axes=[axis], block_size=32, round=rnd)
            assert_bits_equal(got, O.quantize_mx(x, 8, "fp8_e4m3", axes=[axis], block_size=32, round=rnd),
                              "mx axis %d %s" % (axis, rnd))
    assert_bits_equal(elem_gpu(x.to(dev), 9, 8, 2 ** 127 * 255 / 128),
                      O.quantize_elemwise_core(x, 9, 8, 2 ** 127 * 255 / 128), "elementwise")
    with pytest.raises(RuntimeError, match="float16"):
        elem_gpu(x.to(dev), 9, 8, 2 ** 127 * 255 / 128, saturate_normals=True)
    ce.set_exponent_mode("exact")
    try:
        for axis in (-1, 0):
            got = mx_gpu(x.to(dev), 8, "fp4_e2m1", axes=[axis], block_size=32)
            want = mx_gpu(x.float().to(dev), 8, "fp4_e2m1", axes=[axis], block_size=32).half()
            assert got.dtype == torch.float16
            assert_bits_equal(got, want, "mx axis %d" % axis)
        got = elem_gpu(x.to(dev), 5, 4, 448.0, round="even", saturate_normals=True)
        want = elem_gpu(x.float().to(dev), 5, 4, 448.0, round="even", saturate_normals=True).half()
        assert_bits_equal(got, want, "elementwise")
    finally:
        ce.set_exponent_mode("torch")


@pytest.mark.gpu
def test_fp16_dither_with_the_reference_noise_on_the_gpu():
    """round='dither' on fp16 tensors with the noise the reference drew (regenerated on the CPU under
    the stored seed and copied over): the reference's outputs bit for bit."""
    from helpers import dither_cases, reference_noise
    from microxcaling_amd.custom_extensions import funcs
    from microxcaling_amd.formats import _get_format_params
    assert torch.cuda.is_available(), "this test needs a GPU"
    dev = torch.device("cuda:0")
    n = 0
    for kind, name, dtype, case_no, seed, case, x, want in dither_cases():
        if dtype != torch.float16:
            continue
        if kind == "mx" and case[2] > 0 and x.shape[case[1]] % case[2] != 0:
            continue                                  # ragged blocks: tests/test_zt_uncommon_parameters.py
        torch.manual_seed(seed)
        noise = reference_noise(kind, case, x).to(dev)
        if kind == "mx":
            fmt, axis, bs = case
            ebits, mbits, _, max_norm, _ = _get_format_params(fmt)
            got = funcs.quantize_mx_dither_by_tile_func(x.to(dev), noise, 8, ebits, mbits, max_norm, bs,
                                                        axis % x.ndim, False)
        else:
            bits, eb, mn, sat = case
            got = funcs.quantize_elemwise_dither_func(x.to(dev), noise, bits, eb, mn, sat, True)
        torch.cuda.synchronize()
        assert_bits_equal(got, want, "%s %s %d" % (kind, name, case_no))
        n += 1
    assert n == 13


# ---- the layers on fp16 tensors (tests/golden/gen_reference_fp16_layer_vectors.py) ---------------------
def _fp16_layer_fixture():
    import importlib.util
    import os
    spec = importlib.util.spec_from_file_location("gen_reference_fp16_layer_vectors",
                                                  os.path.join(GOLDEN, "gen_reference_fp16_layer_vectors.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return np.load(os.path.join(GOLDEN, "reference_fp16_layer_vectors.npz")), mod


@pytest.mark.parametrize("case", ["mxfp8_bfloat16", "mxfp6_fp16", "mxfp4_floor"])
def test_layers_on_fp16_tensors_reproduce_the_reference(case):
    """linear, bmm, softmax, LayerNorm and RMSNorm on CPU fp16 tensors: forward outputs and every gradient
    as the reference's own layers return them, bit for bit (host-library quantizers + torch's GEMM)."""
    from microxcaling_amd.bmm import bmm
    from microxcaling_amd.layernorm import LayerNorm, RMSNorm
    from microxcaling_amd.linear import linear
    from microxcaling_amd.softmax import softmax
    from microxcaling_amd.specs import finalize_mx_specs
    z, gen = _fp16_layer_fixture()
    t = gen.inputs()
    specs = finalize_mx_specs(dict(dict(gen.SPEC_CASES)[case], quantize_backprop=True, custom_cuda=False))
    want = lambda name: from_bits(z[name], torch.float16)
    threads = torch.get_num_threads()
    torch.set_num_threads(1)                       # the summation order of torch's CPU GEMM the fixtures were written with
    try:
        xi, wi, bi = (t[k].clone().requires_grad_(True) for k in ("x", "w", "b"))
        out = linear(xi, wi, bi, mx_specs=specs)
        out.backward(t["go"])
        for k, v in (("out", out), ("gx", xi.grad), ("gw", wi.grad), ("gb", bi.grad)):
            assert_bits_equal(v, want("linear/%s/%s" % (case, k)), "linear " + k)
        ai, bi2 = t["x"].clone().requires_grad_(True), t["a2"].clone().requires_grad_(True)
        out = bmm(ai, bi2, mx_specs=specs)
        out.backward(t["go"])
        for k, v in (("out", out), ("g1", ai.grad), ("g2", bi2.grad)):
            assert_bits_equal(v, want("bmm/%s/%s" % (case, k)), "bmm " + k)
        si = t["sx"].clone().requires_grad_(True)
        out = softmax(si, dim=-1, mx_specs=specs)
        out.backward(t["sgo"])
        assert_bits_equal(out, want("softmax/%s/out" % case), "softmax out")
        assert_bits_equal(si.grad, want("softmax/%s/gx" % case), "softmax gx")
        for lname, cls in (("layernorm", LayerNorm), ("rmsnorm", RMSNorm)):
            m = cls(64, eps=1e-5, mx_specs=specs).to(torch.float16)
            with torch.no_grad():
                m.weight.copy_(t["nw"])
                m.bias.copy_(t["nb"])
            xi = t["nx"].clone().requires_grad_(True)
            out = m(xi)
            out.backward(t["ngo"])
            for k, v in (("out", out), ("gx", xi.grad), ("gw", m.weight.grad), ("gb", m.bias.grad)):
                assert_bits_equal(v, want("%s/%s/%s" % (lname, case, k)), "%s %s" % (lname, k))
    finally:
        torch.set_num_threads(threads)
