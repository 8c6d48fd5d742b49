"""set_matmul_precision: lets torch run an fp32 matmul through bf16 matrix units when both operands
hold a narrow MX element format that bf16 represents exactly (mx/matmul_precision.py:18-53).
The layers of this package do not need it -- narrow formats go through the packed scaled-MFMA GEMM,
everything else stays in fp32 -- but user code written against the reference may."""
from contextlib import contextmanager

import torch

from .formats import ElemFormat

_NARROW = (ElemFormat.int4, ElemFormat.int2, ElemFormat.fp6_e3m2, ElemFormat.fp6_e2m3, ElemFormat.fp4,
           ElemFormat.fp4_e2m1)


def get_elem_format(inp):
    if inp is None:
        return 'Unknown'
    if type(inp) is str:
        return ElemFormat.from_str(inp)
    return inp


@contextmanager
def set_matmul_precision(a, b, a_elem_format, b_elem_format, force_bf16=False):
    fa, fb = get_elem_format(a_elem_format), get_elem_format(b_elem_format)
    saved_precision = torch.get_float32_matmul_precision()
    saved_reduction = torch.backends.cuda.matmul.allow_bf16_reduced_precision_reduction
    on_gpu = a.device.type == "cuda" and b.device.type == "cuda" and torch.cuda.is_bf16_supported()
    if on_gpu and ((fa in _NARROW and fb in _NARROW) or force_bf16):
        torch.backends.cuda.matmul.allow_bf16_reduced_precision_reduction = False
        torch.set_float32_matmul_precision("medium")
    try:
        yield
    finally:
        torch.set_float32_matmul_precision(saved_precision)
        torch.backends.cuda.matmul.allow_bf16_reduced_precision_reduction = saved_reduction
