"""bfloat softmax: same interface as the reference's mx/softmax.py."""
import torch
import torch.nn as nn
import torch.nn.functional as F

from .specs import apply_mx_specs, get_backwards_mx_specs, mx_assert_test
from .vector_ops import (vec_div, vec_exp, vec_exp2, vec_mul, vec_quantize, vec_reduce_sum,
                         vec_sub)

f_softmax = F.softmax
LN_2_BF16 = 0.69140625           # ln(2) at bfloat16 precision

_DTYPE_CODE = {torch.float32: 0, torch.bfloat16: 2}
MAX_FUSED_ROW = 4096


def _fused_forward(input, dim, mx_specs):
    """The whole forward chain as one kernel launch (mxq_softmax_lastdim), or None when the kernel
    does not cover the case: CPU tensors, another axis than the last, rows longer than 4096 or not
    a multiple of 16 bytes, fp16 tensors, round-half-even to a wide format on a bf16 tensor."""
    from . import _lib, gemm
    from .elemwise_ops import _native_round, elemwise_plan
    if not (gemm.fused_enabled() and input.is_cuda and dim == input.dim() - 1):
        return None
    rnd = mx_specs['round']
    plan = elemwise_plan(mx_specs, rnd)
    if plan[0] == "to_bf16":
        input = input.to(torch.bfloat16)       # the first quantization of the chain does this
        plan = ("identity",)
    if input.dtype not in _DTYPE_CODE:
        return None
    n = input.shape[-1]
    if n == 0 or n > MAX_FUSED_ROW or n % (16 // input.element_size()) != 0:
        return None
    if plan[0] == "identity":
        bits, exp_bits, max_norm, denorm, rmode = 0, 0, 1.0, True, 0
    else:
        _, bits, exp_bits, max_norm, denorm = plan
        rmode = _native_round(rnd)
        if input.dtype == torch.bfloat16 and bits >= 9 and rnd == 'even':
            return None
    if mx_specs.get('softmax_exp2', False):
        exp_mode = 1
    else:
        exp_mode = 2 if mx_specs['vec_use_exp2'] else 0
    x = input.contiguous()
    out = torch.empty_like(x)
    lib = _lib.gpu()
    from .custom_extensions import _flags_value
    with torch.cuda.device(x.device):
        rc = lib.mxq_softmax_lastdim(x.data_ptr(), out.data_ptr(), _DTYPE_CODE[x.dtype],
                                     x.numel() // n, n, bits, exp_bits, max_norm, rmode, int(denorm),
                                     exp_mode, int(bool(mx_specs['vec_use_recip'])), _flags_value(),
                                     torch.cuda.current_stream(x.device).cuda_stream)
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
