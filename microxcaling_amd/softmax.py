"""bfloat softmax: same interface as the reference's mx/softmax.py."""
import torch
import torch.nn as nn
import torch.nn.functional as F

from .specs import apply_mx_specs, get_backwards_mx_specs, mx_assert_test
from .vector_ops import (vec_div, vec_exp, vec_exp2, vec_mul, vec_quantize, vec_reduce_sum,
                         vec_sub)

f_softmax = F.softmax
LN_2_BF16 = 0.69140625           # ln(2) at bfloat16 precision

MAX_FUSED_ROW = 16384


def _fused_forward(input, dim, mx_specs):
    """The whole forward chain as one kernel launch (mxq_softmax_lastdim), or None when the kernel
    does not cover the case: another axis than the last, rows longer than 16384 or not a multiple
    of 16 bytes, and what fused_chain_args excludes."""
    from . import _lib
    from .custom_extensions import _flags_value
    from .elemwise_ops import fused_chain_args
    if dim != input.dim() - 1:
        return None
    args = fused_chain_args(input, mx_specs)
    if args is None:
        return None
    x, code, (bits, exp_bits, max_norm, rmode, denorm) = args
    n = x.shape[-1]
    if n == 0 or n > MAX_FUSED_ROW or n % (16 // x.element_size()) != 0:
        return None
    if mx_specs.get('softmax_exp2', False):
        exp_mode = 1
    else:
        exp_mode = 2 if mx_specs['vec_use_exp2'] else 0
    x = x.contiguous()
    out = torch.empty_like(x)
    lib = _lib.gpu()
    with torch.cuda.device(x.device):
        rc = lib.mxq_softmax_lastdim(x.data_ptr(), out.data_ptr(), code, x.numel() // n, n, bits,
                                     exp_bits, max_norm, rmode, denorm, exp_mode,
                                     int(bool(mx_specs['vec_use_recip'])), _flags_value(),
                                     torch.cuda.current_stream(x.device).cuda_stream)
    _lib.check(rc, lib)
    return out


def _fused_backward(grad_output, output, dim, mx_specs):
    """The backward chain as one kernel launch (mxq_softmax_backward_lastdim), under the same
    conditions as _fused_forward; None otherwise."""
    from . import _lib
    from .custom_extensions import _flags_value
    from .elemwise_ops import fused_chain_args
    if dim != grad_output.dim() - 1:
        return None
    args = fused_chain_args(grad_output, mx_specs)
    if args is None:
        return None
    g, code, (bits, exp_bits, max_norm, rmode, denorm) = args
    n = g.shape[-1]
    if n == 0 or n > MAX_FUSED_ROW or n % (16 // g.element_size()) != 0:
        return None
    if output.dtype != g.dtype or output.shape != g.shape or output.device != g.device:
        return None
    g, y = g.contiguous(), output.contiguous()
    out = torch.empty_like(g)
    lib = _lib.gpu()
    with torch.cuda.device(g.device):
        rc = lib.mxq_softmax_backward_lastdim(g.data_ptr(), y.data_ptr(), out.data_ptr(), code,
                                              g.numel() // n, n, bits, exp_bits, max_norm, rmode, denorm,
                                              int(bool(mx_specs.get('softmax_exp2', False))), _flags_value(),
                                              torch.cuda.current_stream(g.device).cuda_stream)
    _lib.check(rc, lib)
    return out


class SoftmaxFunction(torch.autograd.Function):
    """quantize -> max -> subtract -> exp (or 2^x) -> sum -> divide, re-quantizing after every
    step (mx/softmax.py:20-54; backward 56-88)."""

    @staticmethod
    def forward(ctx, input, dim=None, mx_specs=None, name=None):
        dim = dim + len(input.shape) if dim < 0 else dim
        ctx.dim = dim
        rnd = mx_specs['round']
        fused = _fused_forward(input, dim, mx_specs)
        if fused is not None:
            ctx.save_for_backward(fused)
            ctx.mx_specs = get_backwards_mx_specs(mx_specs)
            return fused
        input = vec_quantize(input, mx_specs=mx_specs)
        max_data, _ = input.max(dim, keepdim=True)
        input = vec_sub(input, max_data, mx_specs=mx_specs, round=rnd)
        if mx_specs.get('softmax_exp2', False):
            output = vec_exp2(input, mx_specs=mx_specs, round=rnd)
        else:
            output = vec_exp(input, mx_specs=mx_specs, round=rnd)
        output_sum = vec_reduce_sum(output, dim, keepdim=True, mx_specs=mx_specs, round=rnd)
        output = vec_div(output, output_sum, mx_specs=mx_specs, round=rnd)
        ctx.save_for_backward(output)
        ctx.mx_specs = get_backwards_mx_specs(mx_specs)
        return output

    @staticmethod
    def backward(ctx, grad_output):
        output, = ctx.saved_tensors
        specs = ctx.mx_specs
        rnd = specs['round']
        fused = _fused_backward(grad_output, output, ctx.dim, specs)
        if fused is not None:
            return (fused, None, None, None)
        grad_output = vec_quantize(grad_output, mx_specs=specs, round=rnd)
        dot = vec_mul(grad_output, output, mx_specs=specs, round=rnd)
        dot = vec_reduce_sum(dot, ctx.dim, keepdim=True, mx_specs=specs, round=rnd)
        grad_input = vec_sub(grad_output, dot, mx_specs=specs, round=rnd)
        grad_input = vec_mul(output, grad_input, mx_specs=specs, round=rnd)
        if specs.get('softmax_exp2', False):
            grad_input = vec_mul(grad_input, LN_2_BF16, mx_specs=specs, round=rnd)
        return (grad_input, None, None, None)


def softmax(input, dim=-1, mx_specs=None, name=None):
    mx_assert_test(mx_specs)
    if mx_specs is None:
        return f_softmax(input, dim=dim)
    mx_specs = apply_mx_specs(mx_specs)
    from .bmm import evaluated, softmax_of_deferred
    out = softmax_of_deferred(input, dim, mx_specs)          # mx.bmm's product, still pending: one kernel for both
    if out is not None:
        return out
    return SoftmaxFunction.apply(evaluated(input), dim, mx_specs, name)


class Softmax(nn.Softmax):
    def __init__(self, dim=None, mx_specs=None, name=None):
        mx_assert_test(mx_specs)
        self.mx_none = mx_specs is None
        self.name = name
        self.mx_specs = apply_mx_specs(mx_specs)
        super().__init__(dim)

    def apply_mx_specs(self, mx_specs):
        self.mx_none = mx_specs is None
        self.mx_specs = apply_mx_specs(mx_specs)

    def append_name(self, postfix):
        self.name += postfix

    def forward(self, input):
        if self.mx_none:
            return super().forward(input)
        return softmax(input, dim=self.dim, mx_specs=self.mx_specs, name=self.name)   # (sees a deferred mx.bmm product)
