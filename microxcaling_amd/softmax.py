"""bfloat softmax: same interface as the reference's mx/softmax.py."""
import torch
import torch.nn as nn
import torch.nn.functional as F

from .specs import apply_mx_specs, get_backwards_mx_specs, mx_assert_test
from .vector_ops import (vec_div, vec_exp, vec_exp2, vec_mul, vec_quantize, vec_reduce_sum,
                         vec_sub)

f_softmax = F.softmax
LN_2_BF16 = 0.69140625           # ln(2) at bfloat16 precision


class SoftmaxFunction(torch.autograd.Function):
    """quantize -> max -> subtract -> exp (or 2^x) -> sum -> divide, re-quantizing after every
    step (mx/softmax.py:20-54; backward 56-88)."""

    @staticmethod
    def forward(ctx, input, dim=None, mx_specs=None, name=None):
        dim = dim + len(input.shape) if dim < 0 else dim
        ctx.dim = dim
        rnd = mx_specs['round']
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
    return SoftmaxFunction.apply(input, dim, mx_specs, name)


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
        return SoftmaxFunction.apply(input, self.dim, self.mx_specs, self.name)
