"""bfloat "vector" ops: a torch op followed by elementwise quantization.  Same names and arguments
as the reference's mx/vector_ops.py:38-130."""
import numpy as np
import torch

from .elemwise_ops import quantize_elemwise_op

# the stock functions, taken now: inject_pyt_ops may later rebind torch.exp / torch.tanh to MX ops
# that are built from the functions below
torch_exp = torch.exp
torch_exp2 = torch.exp2
torch_sqrt = torch.sqrt
torch_tanh = torch.tanh
LN_2_EXACT = 0.69314718056
LOG2_E_BF16 = 1.4453125          # 1 + 2**-2 + 2**-3 + 2**-4 + 2**-7


_ADD, _SUB, _MUL, _DIV = range(4)


def _fused_binary(a, b, op, mx_specs, round):
    """a op b and the elementwise quantizer as one kernel launch (mxq_binary_elemwise), or None when
    the kernel does not stand in for the two steps: no format configured, CPU tensors, operands of
    different shape / dtype (broadcasting, promotion).  Like the quantizer itself, the result is
    not tracked by autograd; the layers call these ops inside their own autograd Functions."""
    if mx_specs is None:
        return None
    ta, tb = torch.is_tensor(a), torch.is_tensor(b)
    if ta and tb:
        if a.shape != b.shape or a.dtype != b.dtype or a.device != b.device:
            return None
        t, other, mode = a, b, 0
    elif ta or tb:
        t, scalar, mode = (a, b, 1) if ta else (b, a, 2)
        if isinstance(scalar, bool) or not isinstance(scalar, (int, float)):
            return None
        other = None
    else:
        return None
    if not t.is_cuda or t.numel() == 0:
        return None
    from .elemwise_ops import elemwise_plan, fused_chain_args
    if elemwise_plan(mx_specs, round)[0] != "quantize":
        return None
    args = fused_chain_args(t, mx_specs, round)
    if args is None:
        return None
    from . import _lib
    from .custom_extensions import _flags_value
    t, code, (bits, exp_bits, max_norm, rmode, denorm) = args
    t = t.contiguous()
    other = None if other is None else other.contiguous()
    out = torch.empty_like(t)
    lib = _lib.gpu()
    with torch.cuda.device(t.device):
        rc = lib.mxq_binary_elemwise(t.data_ptr(), None if other is None else other.data_ptr(),
                                     0.0 if other is not None else float(scalar), mode, out.data_ptr(),
                                     code, t.numel(), op, bits, exp_bits, max_norm, rmode, denorm,
                                     _flags_value(), torch.cuda.current_stream(t.device).cuda_stream)
    _lib.check(rc, lib)
    return out


def vec_quantize(input, mx_specs=None, round=None):
    return quantize_elemwise_op(input, mx_specs=mx_specs, round=round)


def vec_add(a, b, mx_specs=None, round=None):
    fused = _fused_binary(a, b, _ADD, mx_specs, round)
    return fused if fused is not None else quantize_elemwise_op(a + b, mx_specs=mx_specs, round=round)


def vec_sub(a, b, mx_specs=None, round=None):
    fused = _fused_binary(a, b, _SUB, mx_specs, round)
    return fused if fused is not None else quantize_elemwise_op(a - b, mx_specs=mx_specs, round=round)


def vec_mul(a, b, mx_specs=None, round=None):
    fused = _fused_binary(a, b, _MUL, mx_specs, round)
    return fused if fused is not None else quantize_elemwise_op(a * b, mx_specs=mx_specs, round=round)


def vec_recip(input, mx_specs=None, round=None):
    fused = _fused_binary(1., input, _DIV, mx_specs, round)
    return fused if fused is not None else quantize_elemwise_op(1. / input, mx_specs=mx_specs, round=round)


def vec_div(a, b, mx_specs=None, round=None):
    if mx_specs and mx_specs['vec_use_recip']:
        return vec_mul(a, vec_recip(b, mx_specs=mx_specs, round=round), mx_specs=mx_specs,
                       round=round)
    fused = _fused_binary(a, b, _DIV, mx_specs, round)
    return fused if fused is not None else quantize_elemwise_op(a / b, mx_specs=mx_specs, round=round)


def vec_exp2(input, mx_specs=None, round=None):
    return quantize_elemwise_op(torch_exp2(input), mx_specs=mx_specs, round=round)


def vec_exp(input, mx_specs=None, round=None):
    if mx_specs and mx_specs['vec_use_exp2']:
        phi = quantize_elemwise_op(LOG2_E_BF16 * input, mx_specs=mx_specs, round=round)
        return vec_exp2(phi, mx_specs=mx_specs, round=round)
    return quantize_elemwise_op(torch_exp(input), mx_specs=mx_specs, round=round)


def vec_sqrt(input, mx_specs=None, round=None):
    return quantize_elemwise_op(torch_sqrt(input), mx_specs=mx_specs, round=round)


def vec_tanh(input, mx_specs=None, round=None):
    return quantize_elemwise_op(torch_tanh(input), mx_specs=mx_specs, round=round)


def vec_reduce_sum(input, dim, keepdim=False, mx_specs=None, round=None):
    return quantize_elemwise_op(input.sum(dim, keepdim=keepdim), mx_specs=mx_specs, round=round)


def vec_reduce_mean(input, dim, keepdim=False, mx_specs=None, round=None):
    dim = dim if type(dim) is list else [dim]
    denom = np.prod([input.shape[i] for i in dim])          # 1.0 for an empty list
    s = vec_reduce_sum(input, dim, keepdim=keepdim, mx_specs=mx_specs, round=round)
    return vec_div(s, denom, mx_specs=mx_specs, round=round)
