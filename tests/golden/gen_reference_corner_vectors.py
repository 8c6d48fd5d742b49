"""Writes reference_corner_vectors.npz / .json: what the reference's pure-PyTorch CPU path returns
for parameters its own tests hardly touch and that exercise separate branches of a restatement:

  * MX with the wide element formats ``bfloat16`` / ``float16`` and with ``int2`` (mx/formats.py:84-112):
    bfloat16 elements scale every block's maximum into the top binade (emax = 127), where
    floor(log2(x)) evaluated in bf16 reaches 128 for x >= 2**127.5: ``2**128`` is Inf and the element
    comes out NaN (seen on bf16 tensors; fp32's log2 rounds up only next to a power of two, and the
    block maximum then moves the scale); on fp16 tensors the clamp bound does not fit and torch raises;
  * the elementwise quantizer with one exponent bit (``2**(exp_bits-1)`` = 1: min_exp = 0 and a
    quotient that underflows to zero loses its sign in ``sign * |q|``), with integer-like formats
    (exp_bits 0) whose max_norm is 2 or more, and with a clamp bound that the tensor's dtype cannot
    hold (torch.clamp raises).

Run once where the reference checkout exists:
``python tests/golden/gen_reference_corner_vectors.py /root/reference``.  Only inputs and the reference's
outputs are stored; none of the reference's code is."""
import hashlib
import json
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
ROUNDS = ["nearest", "floor", "even"]
DTYPES = {"f32": torch.float32, "bf16": torch.bfloat16, "f16": torch.float16}
MX_WIDE_FORMATS = ["bfloat16", "float16", "int2"]
# (scale_bits, block_size, flush_fp32_subnorms)
MX_SETTINGS = [(8, 32, False), (5, 8, True), (3, 32, False)]
# name -> (bits, exp_bits, max_norm): one exponent bit; integer grids with max_norm >= 2; formats whose
# clamp bound does not fit bf16 / fp16 tensors (a 12-bit mantissa under 8 exponent bits; 2**20)
ELEM_CFG = {
    "e1m2": (4, 1, 1.75), "e1m1": (3, 1, 1.5), "e1m6": (8, 1, 1.984375), "e1m2_wide": (4, 1, 6.0),
    "int_3": (8, 0, 3.0), "int_7p5": (6, 0, 7.5), "int_2": (4, 0, 2.0), "int_448": (5, 0, 448.0),
    "e8m10": (12, 8, 2.0 ** 127 * (2 - 2.0 ** -10)), "e6m3": (5, 6, 2.0 ** 20),
    "e2m1_28": (4, 2, 28.0),
}


def bits_of(t):
    return t.view(torch.int16 if t.element_size() == 2 else torch.int32).numpy().copy()


def digest(t):
    f = t.float().numpy()
    b = bits_of(t)
    nan = np.int16(0x7FC0 if t.dtype == torch.bfloat16 else 0x7E00) if t.element_size() == 2 else np.int32(0x7FC00000)
    return hashlib.sha256(np.ascontiguousarray(np.where(np.isnan(f), nan, b)).tobytes()).hexdigest()


def mx_input(dtype):
    """[rows, 64]: per row a maximum at one exponent of the dtype's range (top binade included), the
    other elements up to 2**-20 below it; rows of zeros, with an Inf, with a NaN."""
    g = torch.Generator().manual_seed(8128)
    lo, hi = {torch.float32: (-140, 127), torch.bfloat16: (-133, 127), torch.float16: (-24, 15)}[dtype]
    rows = []
    for E in list(range(lo, hi + 1, 3)) + [hi - 1, hi]:
        for top in (1.0, 1.9921875, 1.5):
            m = torch.tensor(top, dtype=torch.float64) * 2.0 ** E
            ex = torch.randint(-20, 1, (63,), generator=g).double()
            v = (1 + torch.rand(63, generator=g, dtype=torch.float64)) * torch.exp2(E + ex)
            v = torch.minimum(v, m) * (torch.randint(0, 2, (63,), generator=g) * 2 - 1)
            rows.append(torch.cat([m.reshape(1), v]))
    x = torch.stack(rows).to(torch.float32).to(dtype)
    z = torch.zeros(1, 64, dtype=dtype)
    inf = x[5:6].clone(); inf[0, 3] = float("inf")
    nan = x[7:8].clone(); nan[0, 40] = float("nan")
    return torch.cat([x, z, -z, inf, nan])


def elem_input(dtype):
    if dtype != torch.float32:
        return torch.arange(0, 65536, dtype=torch.int32).to(torch.int16).view(dtype)
    g = torch.Generator().manual_seed(496)
    r = torch.randint(0, 2 ** 31 - 1, (30000,), generator=g, dtype=torch.int64).to(torch.int32).view(torch.float32)
    n = torch.randn(30000, generator=g) * torch.exp2(torch.randint(-12, 12, (30000,), generator=g).float())
    sp = torch.tensor([0.0, float("inf"), float("nan"), 1e-45, 3.4e38, 2.0 ** -126, 2.0 ** -127, 0.25, 0.5, 0.75, 1.0,
                       1.25, 1.5, 1.75, 2.0, 2.5, 3.0, 0.124, 0.126])
    return torch.cat([r, -r, n, sp, -sp])


def main(ref_root):
    sys.path.insert(0, ref_root)
    from mx.mx_ops import _quantize_mx                      # noqa: E402
    from mx.elemwise_ops import _quantize_elemwise_core     # noqa: E402

    out = {}
    meta = {"torch": torch.__version__, "mx_digests": {}, "mx_raises": [], "elem_digests": {},
            "elem_raises": []}
    for dname, dtype in DTYPES.items():
        x = mx_input(dtype)
        out["mx_x." + dname] = bits_of(x)
        for fmt in MX_WIDE_FORMATS:
            for rnd in ROUNDS:
                for (sb, bs, flush) in MX_SETTINGS:
                    key = "%s.%s.%s.%d.%d.%d" % (dname, fmt, rnd, sb, bs, flush)
                    try:
                        y = _quantize_mx(x.clone(), sb, fmt, axes=[-1], block_size=bs, round=rnd,
                                         flush_fp32_subnorms=flush)
                    except RuntimeError:
                        meta["mx_raises"].append(key)        # the clamp bound does not fit the tensor's dtype
                        continue
                    meta["mx_digests"][key] = digest(y)
                    if (sb, rnd) == (8, "nearest") or (fmt, rnd) == ("bfloat16", "even"):
                        out["mx_y." + key] = bits_of(y)
        xe = elem_input(dtype)
        if dtype == torch.float32:
            out["elem_x.f32"] = bits_of(xe)
        for name, (bits, ebits, mx) in ELEM_CFG.items():
            for rnd in ROUNDS:
                for sat in (False, True):
                    for den in (True, False):
                        key = "%s.%s.%s.%d.%d" % (dname, name, rnd, sat, den)
                        try:
                            y = _quantize_elemwise_core(xe.clone(), bits, ebits, mx, round=rnd, saturate_normals=sat,
                                                        allow_denorm=den)
                        except RuntimeError:
                            meta["elem_raises"].append(key)
                            continue
                        meta["elem_digests"][key] = digest(y)
                        if (rnd, sat, den) == ("nearest", False, True) and dname != "f32":
                            out["elem_y." + key] = bits_of(y)
    np.savez_compressed(os.path.join(HERE, "reference_corner_vectors.npz"), **out)
    with open(os.path.join(HERE, "reference_corner_vectors.json"), "w") as f:
        json.dump(meta, f, indent=1, sort_keys=True)
    print("wrote", len(out), "arrays,", len(meta["mx_digests"]), "+", len(meta["elem_digests"]), "digests,",
          len(meta["mx_raises"]), "+", len(meta["elem_raises"]), "raising cases")


if __name__ == "__main__":
    main(sys.argv[1] if len(sys.argv) > 1 else "/root/reference")
