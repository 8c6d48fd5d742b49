"""Writes reference_dither_vectors.npz: outputs of the reference's pure-PyTorch CPU path with
``round='dither'`` (stochastic rounding, mx/elemwise_ops.py:57-59) on seeded inputs under seeded
torch generators.  Run once, in a container where the reference checkout exists:
``python tests/golden/gen_reference_dither_vectors.py /root/reference``.
Only inputs, seeds and the reference's outputs are stored; none of the reference's code is.

The reference draws its noise with torch.rand_like right before the rounding, so a caller that
seeds torch the same way and draws the same number of values of the same dtype gets the same noise:
the fixture pins both the arithmetic of the mode and that this package draws like the reference.
No test of the reference covers this mode.
"""
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
MX_CASES = [("fp8_e4m3", -1, 32), ("fp8_e5m2", 0, 32), ("fp6_e3m2", -1, 32), ("fp6_e2m3", 0, 16),
            ("fp4_e2m1", -1, 32), ("int8", -1, 0), ("int4", 0, 32),
            # blocks that do not divide the axis: the reference draws its noise for the padded tensor
            ("fp8_e4m3", -1, 64), ("fp6_e2m3", 0, 5), ("int8", -1, 7)]
ELEM_CASES = [(9, 8, 2 ** 127 * 255 / 128, False), (12, 5, 65504.0, False), (12, 5, 65504.0, True),
              (5, 4, 448.0, True), (8, 0, 127 / 64, False), (5, 8, 2 ** 127 * 1.875, False)]


def inputs(dtype):
    g = torch.Generator().manual_seed(4242)
    span = 12 if dtype == torch.float16 else 24         # fp16 holds 2**-24 .. 2**16
    x = torch.randn(64, 96, generator=g) * torch.exp2(torch.randint(-span, span, (64, 96), generator=g).float())
    x = x.to(dtype)
    x[0, :8] = torch.tensor([0.0, -0.0, float("inf"), float("-inf"), float("nan"), 1e-39, 3e38, -1e-41]).to(dtype)
    x[1] = 0.0                                   # a block of zeros
    x[2, :32] *= 1e-30                           # tiny block
    return x


def raw(t):
    return (t.view(torch.int32) if t.dtype == torch.float32 else t.view(torch.int16)).numpy().copy()


def main(ref_root):
    sys.path.insert(0, ref_root)
    from mx.mx_ops import _quantize_mx                      # noqa: E402
    from mx.elemwise_ops import _quantize_elemwise_core     # noqa: E402
    out = {}
    for name, dtype in (("f32", torch.float32), ("bf16", torch.bfloat16), ("f16", torch.float16)):
        x = inputs(dtype)
        out["x_" + name] = raw(x)
        for n, (fmt, axis, bs) in enumerate(MX_CASES):
            torch.manual_seed(1000 + n)
            y = _quantize_mx(x.clone(), 8, fmt, axes=[axis], block_size=bs, round="dither", custom_cuda=False)
            out["mx_%s_%d" % (name, n)] = raw(y)
        for n, (bits, eb, mn, sat) in enumerate(ELEM_CASES):
            torch.manual_seed(2000 + n)
            y = _quantize_elemwise_core(x.clone(), bits, eb, mn, round="dither", saturate_normals=sat,
                                        custom_cuda=False)
            out["elem_%s_%d" % (name, n)] = raw(y)
    np.savez_compressed(os.path.join(HERE, "reference_dither_vectors.npz"), **out)
    print("wrote %d arrays" % len(out))


if __name__ == "__main__":
    main(sys.argv[1] if len(sys.argv) > 1 else "/root/reference")
