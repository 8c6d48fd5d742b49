"""ctypes access to the C restatement (libmxq_oracle.so).  TEST INFRASTRUCTURE ONLY."""
import ctypes
import os

import torch

from . import build_oracle
from .mx_oracle import format_params

_lib = None
_DT = {torch.float32: 0, torch.float16: 1, torch.bfloat16: 2}


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(build_oracle.LIB):
            build_oracle.build(verbose=False)
        _lib = ctypes.CDLL(build_oracle.LIB)
        i64, ci, cf, vp = ctypes.c_int64, ctypes.c_int, ctypes.c_float, ctypes.c_void_p
        _lib.oracle_quantize_elemwise.argtypes = [vp, vp, ci, i64, ci, ci, cf, ci, ci, ci]
        _lib.oracle_quantize_elemwise.restype = None
        _lib.oracle_quantize_mx.argtypes = [vp, vp, ci, i64, i64, i64, ci, ci, ci, ci, cf, i64, ci, ci]
        _lib.oracle_quantize_mx.restype = None
    return _lib


_RMODE = {"nearest": 0, "floor": 1, "even": 2}


def _clamp_bound_must_fit(dtype, max_norm):
    """torch.clamp converts its bounds to the tensor dtype and refuses one that overflows it
    (mx/elemwise_ops.py:154 on an fp16 / bf16 tensor)."""
    if dtype in (torch.float16, torch.bfloat16) and max_norm > torch.finfo(dtype).max:
        raise RuntimeError("value cannot be converted to type %s without overflow" % dtype)


def quantize_elemwise_core(A, bits, exp_bits, max_norm, round="nearest", saturate_normals=False,
                           allow_denorm=True):
    A = A.contiguous()
    if saturate_normals or exp_bits == 0:
        _clamp_bound_must_fit(A.dtype, max_norm)
    out = torch.empty_like(A)
    lib().oracle_quantize_elemwise(A.data_ptr(), out.data_ptr(), _DT[A.dtype], A.numel(), bits,
                                   exp_bits, max_norm, _RMODE[round], int(saturate_normals),
                                   int(allow_denorm))
    return out


def quantize_mx(A, scale_bits, elem_format, axes, block_size=0, round="nearest",
                flush_fp32_subnorms=False):
    A = A.contiguous()
    (axis,) = [axes] if isinstance(axes, int) else axes
    for _ in range(2):             # the reference normalizes a negative axis twice (mx/mx_ops.py:193-194, 105)
        axis = axis + A.ndim if axis < 0 else axis
    if not 0 <= axis < A.ndim:
        raise IndexError("axis out of range for a tensor of %d dimensions" % A.ndim)
    pre = 1
    for n in A.shape[:axis]:
        pre *= n
    post = 1
    for n in A.shape[axis + 1:]:
        post *= n
    ebits, mbits, emax, max_norm, _ = format_params(elem_format)
    _clamp_bound_must_fit(A.dtype, max_norm)            # elements are saturated (mx/mx_ops.py:287-290)
    out = torch.empty_like(A)
    lib().oracle_quantize_mx(A.data_ptr(), out.data_ptr(), _DT[A.dtype], pre, A.shape[axis], post,
                             scale_bits, ebits, mbits, emax, max_norm, block_size,
                             int(flush_fp32_subnorms), _RMODE[round])
    return out
