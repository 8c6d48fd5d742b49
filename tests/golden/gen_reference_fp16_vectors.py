"""Writes reference_fp16_vectors.npz / .json: what the reference's pure-PyTorch CPU path
(``custom_cuda=False``) returns for float16 *tensors*, where it evaluates every op in fp16
(mx/mx_ops.py:265-292, mx/elemwise_ops.py:127-163).  Run once, in a container where the reference
checkout exists:  ``python tests/golden/gen_reference_fp16_vectors.py /root/reference``.
Only inputs and the reference's outputs are stored; none of the reference's code is.

What these cases are chosen to catch:
  * floor(log2(x)) evaluated in fp16 rounds up just below powers of two (top 1..11 codes of a
    binade) -- block maxima and elements inside and beside those zones;
  * 2**shared_exp is an fp16 number: Inf from 2**16, zero below 2**-24 -- blocks whose scale
    overflows or underflows come out as NaN, all-zero blocks included (log2(0) = -inf);
  * x / 2**se can be an fp16 subnormal and rounds there before the element rounding sees it;
  * "+ 0.5" has no room from 1024 on (wide element formats), products overflow at 65520;
  * the clamp bound is cast to fp16 (the reference raises when it does not fit).
"""
import hashlib
import json
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
MX_FORMATS = ["fp8_e4m3", "fp8_e5m2", "fp6_e3m2", "fp6_e2m3", "fp4_e2m1", "int8", "int4"]
ROUNDS = ["nearest", "floor", "even"]
BF16_MAX = 2 ** 127 * 255 / 128
# name -> (bits, exp_bits, max_norm) of the elementwise cases
ELEM_CFG = {"bf16": (9, 8, BF16_MAX), "fp16": (12, 5, 65504.0), "e4m3": (5, 4, 448.0),
            "e5m2": (4, 5, 57344.0), "wide": (20, 5, 65504.0), "e6m5": (7, 6, 65504.0),
            "int8": (8, 0, 1.984375)}
# block maxima of the exhaustive sweep: (exponent, top fraction bits of the fp16 code)
EXHAUSTIVE_MAXIMA = [(-24, 0), (-20, 0), (-17, 0), (-16, 0), (-14, 0), (-9, 0x3FF), (-3, 0), (0, 0),
                     (0, 0x3FF), (1, 0), (5, 0x3F0), (10, 0), (15, 0), (15, 0x3FF)]


def bits16(t):
    return t.view(torch.int16).numpy().copy()


def digest(t):
    """sha256 over the fp16 bit patterns with every NaN mapped to the canonical quiet NaN."""
    b = np.where(np.isnan(t.float().numpy()), np.int16(0x7E00), bits16(t))
    return hashlib.sha256(np.ascontiguousarray(b).tobytes()).hexdigest()


def all_fp16_codes():
    return torch.arange(0, 65536, dtype=torch.int32).to(torch.int16).view(torch.float16)


def fp16_value(exp, frac):
    """The fp16 number 2**exp * (1 + frac / 1024); below 2**-14 the subnormal 2**exp (frac ignored)."""
    if exp < -14:
        return 2.0 ** exp
    code = ((exp + 15) << 10) | frac
    return torch.tensor([code], dtype=torch.int16).view(torch.float16).float().item()


def exhaustive_block(exp, frac):
    """[n, 32] fp16: the maximum first, then every finite fp16 code not above it, 31 per row."""
    codes = all_fp16_codes()
    finite = codes[torch.isfinite(codes.float())]
    M = fp16_value(exp, frac)
    sel = finite[finite.float().abs() <= M]
    n = (sel.numel() + 30) // 31 * 31
    body = torch.cat([sel, torch.zeros(n - sel.numel(), dtype=torch.float16)]).view(-1, 31)
    return torch.cat([torch.full((body.shape[0], 1), M, dtype=torch.float16), body], dim=1)


def fp16_block_cases():
    """[n_blocks, 32] fp16 rows: a maximum M (every exponent of the dtype, plain and top-of-binade
    fractions) followed by 31 values not above it -- all-ones fractions, near-top fractions, random."""
    g = torch.Generator().manual_seed(1616)
    rows = []
    for E in range(-24, 16):
        for top in (0, 0x3FF, 0x3FB, 0x3F5, 0x2A0):
            if E < -14 and top:
                continue
            M = fp16_value(E, top)
            for rep in range(3):
                ex = (torch.randint(-13, 1, (31,), generator=g) + E).clamp(min=-24)
                man = torch.randint(0, 1024, (31,), generator=g)
                if rep == 0:
                    man[:] = 1023
                if rep == 1:
                    man = torch.randint(1008, 1024, (31,), generator=g)
                sgn = torch.randint(0, 2, (31,), generator=g)
                normal = ((sgn << 15) | ((ex + 15).clamp(min=0) << 10) | man)
                sub = (sgn << 15) | (man >> (-14 - ex).clamp(min=0, max=10)).clamp(min=1)
                c = torch.where(ex < -14, sub, normal)
                v = c.to(torch.int16).view(torch.float16).float()
                v = torch.where(v.abs() > M, torch.full_like(v, M) * torch.sign(v), v)
                rows.append(torch.cat([torch.tensor([M]), v]))
    # blocks of zeros, of one sign of zero, with an Inf and with a NaN
    z = torch.zeros(32)
    rows += [z, -z, torch.cat([torch.tensor([float("inf")]), torch.ones(31)]),
             torch.cat([torch.tensor([float("nan")]), torch.ones(31)]),
             torch.cat([torch.tensor([-float("inf"), 0.0]), -torch.ones(30)])]
    return torch.stack(rows).to(torch.float16)


def main(ref_root):
    sys.path.insert(0, ref_root)
    from mx.mx_ops import _quantize_mx                      # noqa: E402
    from mx.elemwise_ops import _quantize_elemwise_core     # noqa: E402

    out = {}
    meta = {"torch": torch.__version__, "mx_digests": {}, "elem_digests": {}, "elem_raises": []}

    # 1. block cases, stored in full
    xb = fp16_block_cases()
    out["mx_x"] = bits16(xb)
    for fmt in MX_FORMATS:
        for rnd in ROUNDS:
            y = _quantize_mx(xb.clone(), 8, fmt, axes=[-1], block_size=32, round=rnd)
            out["mx_y.%s.%s" % (fmt, rnd)] = bits16(y)
    y = _quantize_mx(xb.t().contiguous(), 5, "fp8_e4m3", axes=[0], block_size=32, round="even",
                     flush_fp32_subnorms=True)
    out["mx_y.t.fp8_e4m3.even.sb5.flush"] = bits16(y)
    y = _quantize_mx(xb.clone(), 8, "fp6_e2m3", axes=[-1], block_size=32, round="nearest", flush_fp32_subnorms=True)
    out["mx_y.fp6_e2m3.nearest.flush"] = bits16(y)
    y = _quantize_mx(xb.clone(), 4, "int8", axes=[-1], block_size=8, round="floor")
    out["mx_y.int8.floor.sb4.bs8"] = bits16(y)
    y = _quantize_mx(xb[:, :24].contiguous(), 8, "fp4_e2m1", axes=[-1], block_size=16, round="even")
    out["mx_y.fp4_e2m1.even.ragged24.bs16"] = bits16(y)

    # 2. every finite fp16 code as an element under a spread of block maxima: digests, two stored
    for (exp, frac) in EXHAUSTIVE_MAXIMA:
        blk = exhaustive_block(exp, frac)
        for fmt in MX_FORMATS:
            for rnd in ROUNDS:
                for sb in (8, 5):
                    y = _quantize_mx(blk.clone(), sb, fmt, axes=[-1], block_size=32, round=rnd)
                    meta["mx_digests"]["%d.%d.%s.%s.%d" % (exp, frac, fmt, rnd, sb)] = digest(y)
    out["mx_exh_y.0.1023.fp8_e4m3.nearest.8"] = bits16(
        _quantize_mx(exhaustive_block(0, 0x3FF), 8, "fp8_e4m3", axes=[-1], block_size=32, round="nearest"))
    out["mx_exh_y.15.1023.fp8_e5m2.floor.8"] = bits16(
        _quantize_mx(exhaustive_block(15, 0x3FF), 8, "fp8_e5m2", axes=[-1], block_size=32, round="floor"))

    # 3. the elementwise quantizer on every fp16 code
    codes = all_fp16_codes()
    for name, (bits, ebits, mx) in ELEM_CFG.items():
        for rnd in ROUNDS:
            for sat in (False, True):
                for den in (True, False):
                    key = "%s.%s.%d.%d" % (name, rnd, sat, den)
                    try:
                        y = _quantize_elemwise_core(codes.clone(), bits, ebits, mx, round=rnd,
                                                    saturate_normals=sat, allow_denorm=den)
                    except RuntimeError:
                        meta["elem_raises"].append(key)      # the clamp bound does not fit fp16
                        continue
                    meta["elem_digests"][key] = digest(y)
                    if (rnd, sat, den) == ("nearest", False, True) or (name, rnd, den) == ("fp16", "even", True):
                        out["elem_y." + key] = bits16(y)

    np.savez_compressed(os.path.join(HERE, "reference_fp16_vectors.npz"), **out)
    with open(os.path.join(HERE, "reference_fp16_vectors.json"), "w") as f:
        json.dump(meta, f, indent=1, sort_keys=True)
    print("wrote", len(out), "arrays,", len(meta["mx_digests"]), "+", len(meta["elem_digests"]), "digests,",
          len(meta["elem_raises"]), "raising cases")


if __name__ == "__main__":
    main(sys.argv[1] if len(sys.argv) > 1 else "/root/reference")
