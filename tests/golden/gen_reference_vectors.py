"""Writes the golden fixtures in this folder by running the reference's pure-PyTorch CPU path
(``custom_cuda=False``) on seeded inputs.  Run once, in a container where the reference checkout
exists:  ``python tests/golden/gen_reference_vectors.py /root/reference``.
Only inputs and the reference's outputs are stored; none of the reference's code is.

Covered here are the behaviours no literal vector of the reference's own tests pins:
  * bf16 (and fp16) *tensors* through ``_quantize_mx`` -- every op rounds to the tensor dtype;
  * the floor(log2(x)) round-up zone just below powers of two (shared exponent in every rounding
    mode, element exponent in 'floor' mode), fp32 and bf16;
  * ``_quantize_elemwise_core`` on fp32 specials (Inf/NaN/subnormals/near FLT_MAX).
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


def bits16(t):
    return t.view(torch.int16).numpy().copy()


def bits32(t):
    return t.view(torch.int32).numpy().copy()


def digest(t):
    """sha256 over the output bit patterns with every NaN mapped to the canonical quiet NaN."""
    if t.dtype == torch.float32:
        b = np.where(np.isnan(t.numpy()), np.int32(0x7FC00000), bits32(t))
    else:
        b = np.where(np.isnan(t.float().numpy()), np.int16(0x7FC0), bits16(t))
    return hashlib.sha256(np.ascontiguousarray(b).tobytes()).hexdigest()


def all_bf16_codes():
    return torch.arange(0, 65536, dtype=torch.int32).to(torch.int16).view(torch.bfloat16)


def bf16_block_cases():
    """[n_blocks, 32] bf16: for a spread of block maxima M (powers of two and top-of-binade values,
    subnormal to huge), rows made of M followed by 31 probe values not exceeding M in magnitude.
    Probes sweep every mantissa code in the binades that matter for the element format."""
    g = torch.Generator().manual_seed(1234)
    rows = []
    max_exps = list(range(-133, -118)) + list(range(-20, 21)) + list(range(110, 128))
    for E in max_exps:
        for top in (0, 0x7F, 0x7B, 0x50):
            if E < -126:
                code = (1 << (E + 133)) | ((top << (E + 133)) >> 7 if top else 0)
                code = max(1, min(code, 0x7F))
            else:
                code = ((E + 127) << 7) | top
            M = torch.tensor([code], dtype=torch.int16).view(torch.bfloat16).float().item()
            for rep in range(3):
                # random bf16 codes scaled under M: exponents from E-14 .. E, random sign/mantissa
                ex = torch.randint(-14, 1, (31,), generator=g) + E
                ex = ex.clamp(min=-133)
                man = torch.randint(0, 128, (31,), generator=g)
                if rep == 0:
                    man[:] = 127                       # all-ones mantissas (0.5 - 2^-9 style ties)
                if rep == 1:
                    man = torch.randint(120, 128, (31,), generator=g)
                sgn = torch.randint(0, 2, (31,), generator=g)
                be = (ex + 127).clamp(min=0)
                c = (sgn << 15) | (be << 7) | man
                sub = ex < -126                        # bf16 subnormals: mantissa only
                c = torch.where(sub, (sgn << 15) | (man >> (-126 - ex).clamp(min=0, max=7)), c)
                v = c.to(torch.int16).view(torch.bfloat16).float()
                v = torch.where(v.abs() > M, torch.full_like(v, M) * torch.sign(v), v)
                rows.append(torch.cat([torch.tensor([M]), v]))
    return torch.stack(rows).to(torch.bfloat16)


def fp32_zone_cases():
    """[n_blocks, 32] fp32 blocks whose maximum, or whose elements after scaling, sit within a few
    ulps below a power of two."""
    g = torch.Generator().manual_seed(4321)
    rows = []
    for E in list(range(-149, -120, 2)) + list(range(-12, 13)) + list(range(101, 128, 3)):
        for back in (0, 1, 2, 5, 6, 11, 22, 44, 45, 89):
            if E >= -126:
                code = ((E + 127) << 23) + (1 << 23) - 1 - back
            else:
                code = (1 << (E + 150)) - 1 - back
            if code <= 0:
                continue
            M = torch.tensor([code], dtype=torch.int32).view(torch.float32)
            # elements: M scaled down by powers of two (stay in the zone after division by the
            # scale) mixed with random values below M
            scl = 2.0 ** -torch.randint(0, 12, (31,), generator=g).float()
            v = M * scl
            rnd = (torch.rand(31, generator=g) * 2 - 1) * M
            pick = torch.rand(31, generator=g) < 0.5
            v = torch.where(pick, v * torch.sign(rnd), rnd)
            rows.append(torch.cat([M, v]))
    return torch.stack(rows)


def fp32_special_elems():
    g = torch.Generator().manual_seed(99)
    parts = []
    # top-of-binade codes for every exponent
    for be in range(0, 255):
        base = (be << 23) + (1 << 23)
        c = base - 1 - torch.tensor([0, 1, 2, 3, 5, 6, 11, 12, 22, 23, 44, 45, 88, 89])
        parts.append(c[c > 0])
    c = torch.cat(parts)
    vals = c.to(torch.int32).view(torch.float32)
    rnd = torch.randint(0, 2 ** 31 - 1, (4000,), generator=g, dtype=torch.int64)
    rnd = rnd.to(torch.int32).view(torch.float32)
    spec = torch.tensor([0.0, -0.0, float("inf"), -float("inf"), float("nan"),
                         3.4028234663852886e38, -3.4028234663852886e38, 1e-45, -1e-45,
                         65504., 65519., 65520., 65535., 65536., 2 ** -14, 2 ** -24, 2 ** -25,
                         2 ** -126, 2 ** -133, 2 ** -134])
    v = torch.cat([vals, rnd, spec])
    return torch.cat([v, -v])


def main(ref_root):
    sys.path.insert(0, ref_root)
    from mx.mx_ops import _quantize_mx                      # noqa: E402
    from mx.elemwise_ops import _quantize_elemwise_core     # noqa: E402

    out = {}
    meta = {"torch": torch.__version__, "digests": {}}

    # 1. bf16 tensors through _quantize_mx
    xb = bf16_block_cases()
    out["mx_bf16_x"] = bits16(xb)
    for fmt in MX_FORMATS:
        for rnd in ROUNDS:
            y = _quantize_mx(xb.clone(), 8, fmt, axes=[-1], block_size=32, round=rnd)
            out["mx_bf16_y.%s.%s" % (fmt, rnd)] = bits16(y)
    # along axis 0 of the transposed tensor, scale_bits 5, flush
    y = _quantize_mx(xb.t().contiguous(), 5, "fp8_e4m3", axes=[0], block_size=32, round="even",
                     flush_fp32_subnorms=True)
    out["mx_bf16_y.t.fp8_e4m3.even.sb5.flush"] = bits16(y)

    # 2. exhaustive bf16 codes as elements, several block maxima, hashed (+ stored for two cases)
    codes = all_bf16_codes()
    finite = codes[torch.isfinite(codes.float())]
    digests = {}
    for Mexp in (-130, -126, -100, -3, 0, 1, 5, 60, 120, 127):
        M = 2.0 ** Mexp
        sel = finite[finite.float().abs() <= M]
        n = (sel.numel() + 30) // 31 * 31
        pad = torch.zeros(n - sel.numel(), dtype=torch.bfloat16)
        body = torch.cat([sel, pad]).view(-1, 31)
        blk = torch.cat([torch.full((body.shape[0], 1), M, dtype=torch.bfloat16), body], dim=1)
        for fmt in MX_FORMATS:
            for rnd in ROUNDS:
                y = _quantize_mx(blk.clone(), 8, fmt, axes=[-1], block_size=32, round=rnd)
                digests["%d.%s.%s" % (Mexp, fmt, rnd)] = digest(y)
    meta["bf16_exhaustive_digests"] = digests

    # 3. fp32 zone blocks
    xz = fp32_zone_cases()
    out["mx_fp32_zone_x"] = bits32(xz)
    for fmt in MX_FORMATS:
        for rnd in ROUNDS:
            y = _quantize_mx(xz.clone(), 8, fmt, axes=[-1], block_size=32, round=rnd)
            out["mx_fp32_zone_y.%s.%s" % (fmt, rnd)] = bits32(y)

    # 4. elementwise core on fp32 specials and on bf16 tensors
    xe = fp32_special_elems()
    out["elem_fp32_x"] = bits32(xe)
    for name, (bits, ebits, mx) in {"bf16": (9, 8, 2 ** 127 * 255 / 128),
                                     "fp16": (12, 5, 65504.0),
                                     "bf12": (5, 8, 2 ** 127 * 15 / 8)}.items():
        for rnd in ROUNDS:
            for sat in (False, True):
                for den in (True, False):
                    y = _quantize_elemwise_core(xe.clone(), bits, ebits, mx, round=rnd,
                                                saturate_normals=sat, allow_denorm=den)
                    key = "elem_fp32_y.%s.%s.%d.%d" % (name, rnd, sat, den)
                    meta["digests"][key] = digest(y)
                    if (sat, den) == (False, True) or (name, rnd) == ("bf16", "floor"):
                        out[key] = bits32(y)
    xb16 = all_bf16_codes()
    out["elem_bf16_x"] = bits16(xb16)
    for name, (bits, ebits, mx) in {"bf16": (9, 8, 2 ** 127 * 255 / 128),
                                     "fp16": (12, 5, 65504.0),
                                     "e4m3": (5, 4, 448.0)}.items():
        for rnd in ROUNDS:
            for sat in (False, True):
                y = _quantize_elemwise_core(xb16.clone(), bits, ebits, mx, round=rnd,
                                            saturate_normals=sat, allow_denorm=True)
                key = "elem_bf16_y.%s.%s.%d" % (name, rnd, sat)
                meta["digests"][key] = digest(y)
                if (name, rnd, sat) in (("bf16", "nearest", False), ("fp16", "floor", False),
                                        ("e4m3", "even", True)):
                    out[key] = bits16(y)

    np.savez_compressed(os.path.join(HERE, "reference_vectors.npz"), **out)
    with open(os.path.join(HERE, "reference_vectors.json"), "w") as f:
        json.dump(meta, f, indent=1, sort_keys=True)
    print("wrote", len(out), "arrays")


if __name__ == "__main__":
    main(sys.argv[1] if len(sys.argv) > 1 else "/root/reference")
