"""Parameters the reference's own tests hardly use and that take separate branches here: MX with the
wide element formats (bfloat16, float16) and int2, the elementwise quantizer with one exponent bit,
with integer grids whose max_norm is 2 or more, and with clamp bounds the tensor's dtype cannot hold.
tests/golden/gen_reference_corner_vectors.py stored what the reference's pure path returns
(mx/mx_ops.py:265-292, mx/elemwise_ops.py:127-163).  The same bodies run against both oracles, the
host library and (marked gpu) the HIP kernels through the C ABI."""
import hashlib
import importlib.util
import json
import os

import numpy as np
import pytest
import torch

from helpers import GOLDEN, PackageImpl, assert_bits_equal, canon_bits, from_bits
from oracle import c_oracle as C
from oracle import mx_oracle as O

ORACLES = [pytest.param(O, id="torch"), pytest.param(C, id="c"),
           pytest.param(PackageImpl("cpu"), id="host_library"),
           pytest.param(PackageImpl("cuda"), id="hip", marks=pytest.mark.gpu)]

_golden = None


def corner_golden():
    global _golden
    if _golden is None:
        spec = importlib.util.spec_from_file_location("gen_reference_corner_vectors",
                                                      os.path.join(GOLDEN, "gen_reference_corner_vectors.py"))
        mod = importlib.util.module_from_spec(spec)
        spec.loader.exec_module(mod)
        with open(os.path.join(GOLDEN, "reference_corner_vectors.json")) as f:
            meta = json.load(f)
        _golden = (np.load(os.path.join(GOLDEN, "reference_corner_vectors.npz")), meta, mod)
    return _golden


def _digest(t):
    return hashlib.sha256(np.ascontiguousarray(canon_bits(t)).tobytes()).hexdigest()


@pytest.mark.parametrize("orc", ORACLES)
@pytest.mark.parametrize("dname", ["f32", "bf16", "f16"])
def test_golden_mx_wide_element_formats(orc, dname):
    """MX with element formats bfloat16, float16 and int2, block maxima over the dtype's whole exponent
    range.  bfloat16 elements put every block's maximum into binade 127, where floor(log2(x)) evaluated in
    bf16 gives 128 from 2**127.5 on and 2**128 = Inf turns the element into NaN (bf16 tensors); on fp16
    tensors bfloat16 elements raise (the clamp bound does not fit)."""
    z, meta, gen = corner_golden()
    dtype = gen.DTYPES[dname]
    x = from_bits(z["mx_x." + dname], dtype)
    n = 0
    for fmt in gen.MX_WIDE_FORMATS:
        for rnd in gen.ROUNDS:
            for (sb, bs, flush) in gen.MX_SETTINGS:
                key = "%s.%s.%s.%d.%d.%d" % (dname, fmt, rnd, sb, bs, flush)
                call = lambda: orc.quantize_mx(x.clone(), sb, fmt, axes=[-1], block_size=bs, round=rnd,
                                               flush_fp32_subnorms=flush)
                if key in meta["mx_raises"]:
                    with pytest.raises(RuntimeError):
                        call()
                    continue
                y = call()
                if "mx_y." + key in z.files:
                    assert_bits_equal(y, from_bits(z["mx_y." + key], dtype), key)
                assert _digest(y) == meta["mx_digests"][key], key
                n += 1
    assert n == (18 if dname == "f16" else 27)


@pytest.mark.parametrize("orc", ORACLES)
@pytest.mark.parametrize("dname", ["f32", "bf16", "f16"])
def test_golden_elementwise_uncommon_formats(orc, dname):
    """One exponent bit (a quotient that underflows to zero loses its sign), integer grids with max_norm
    of 2 and more, max_norm above the format's own grid, clamp bounds beyond the tensor's dtype (raise):
    every bf16 / fp16 code, and 90 000 fp32 values."""
    z, meta, gen = corner_golden()
    dtype = gen.DTYPES[dname]
    x = from_bits(z["elem_x.f32"], dtype) if dname == "f32" else gen.elem_input(dtype)
    n = raised = 0
    for name, (bits, ebits, mx) in gen.ELEM_CFG.items():
        for rnd in gen.ROUNDS:
            for sat in (False, True):
                for den in (True, False):
                    key = "%s.%s.%s.%d.%d" % (dname, name, rnd, sat, den)
                    call = lambda: orc.quantize_elemwise_core(x.clone(), bits, ebits, mx, round=rnd,
                                                              saturate_normals=sat, allow_denorm=den)
                    if key in meta["elem_raises"]:
                        with pytest.raises(RuntimeError):
                            call()
                        raised += 1
                        continue
                    y = call()
                    if "elem_y." + key in z.files:
                        assert_bits_equal(y, from_bits(z["elem_y." + key], dtype), key)
                    assert _digest(y) == meta["elem_digests"][key], key
                    n += 1
    assert (n, raised) == {"f32": (132, 0), "bf16": (126, 6), "f16": (120, 12)}[dname]


def test_one_exponent_bit_drops_the_sign_of_an_underflowed_quotient():
    """exp_bits = 1: the reference computes sign(x) * round(|x| / 2**e) * 2**e, and where the quotient
    itself underflows to zero the product is taken with a zero of the sign's own making: among negative
    inputs that quantize to zero both +0 and -0 occur.  Host library against the stored reference bits."""
    z, meta, gen = corner_golden()
    x = gen.elem_input(torch.bfloat16)
    want = from_bits(z["elem_y.bf16.e1m2.nearest.0.1"], torch.bfloat16)
    got = PackageImpl("cpu").quantize_elemwise_core(x.clone(), 4, 1, 1.75)
    neg_zero_in = (x.float() < 0) & (want.float() == 0)
    assert int(neg_zero_in.sum()) > 1000
    signs = canon_bits(want)[neg_zero_in.numpy()]
    assert {int(v) & 0xFFFF for v in np.unique(signs)} == {0x0000, 0x8000}     # both signs of zero occur
    assert_bits_equal(got, want, "e1m2")


@pytest.mark.gpu
def test_dither_with_ragged_blocks_on_the_gpu():
    """round='dither' where the block size does not divide the axis (three stored settings x three dtypes):
    with the noise the reference drew -- for the tensor padded to whole blocks -- regenerated on the CPU and
    copied over, the kernel gives the reference's outputs bit for bit; and the public call on a GPU tensor
    draws a padded-shape noise tensor of its own and returns a finite, correctly shaped result."""
    from helpers import dither_cases, reference_noise
    from microxcaling_amd.custom_extensions import funcs
    from microxcaling_amd.formats import _get_format_params
    from microxcaling_amd.mx_ops import _quantize_mx
    assert torch.cuda.is_available(), "this test needs a GPU"
    dev = torch.device("cuda:0")
    n = 0
    for kind, name, dtype, case_no, seed, case, x, want in dither_cases():
        if kind != "mx" or case[2] <= 0 or x.shape[case[1]] % case[2] == 0:
            continue
        fmt, axis, bs = case
        torch.manual_seed(seed)
        noise = reference_noise(kind, case, x).to(dev)
        ebits, mbits, _, max_norm, _ = _get_format_params(fmt)
        got = funcs.quantize_mx_dither_by_tile_func(x.to(dev), noise, 8, ebits, mbits, max_norm, bs, axis % x.ndim, False)
        torch.cuda.synchronize()
        assert_bits_equal(got, want, "%s %s %d" % (kind, name, case_no))
        y = _quantize_mx(torch.ones(5, 70, dtype=dtype, device=dev), 8, fmt, axes=[axis], block_size=bs, round="dither")
        assert y.shape == (5, 70) and bool(torch.isfinite(y.float()).all())
        n += 1
    assert n == 9
