"""Adaptive average pooling (N, C, H, W) -> (N, C, oH, oW) with quantized means: same interface as
the reference's mx/adaptive_avg_pooling.py."""
import math

import torch
import torch.nn as nn
import torch.nn.functional as F

from .specs import apply_mx_specs, get_backwards_mx_specs, mx_assert_test
from .vector_ops import vec_add, vec_reduce_mean

f_adaptive_avg_pool2d = F.adaptive_avg_pool2d


def start_index(a, b, c):
    return math.floor((float(a) * float(c)) / b)


def end_index(a, b, c):
    return math.ceil((float(a + 1) * float(c)) / b)


def _windows(out_size, in_size):
    """(output index, first input index, one past the last) of every pooling window along one axis."""
    return [(o, start_index(o, out_size, in_size), end_index(o, out_size, in_size))
            for o in range(out_size)]


def _resolve_output_size(output_size, H, W):
    if isinstance(output_size, tuple) and len(output_size) == 2:
        return (output_size[0] or H), (output_size[1] or W)          # None keeps the input size
    if isinstance(output_size, int):
        return output_size, output_size
    if output_size is None:
        return H, W
    raise ValueError('expected 1D or 2D output_size (got {}D output_size)'.format(len(output_size)))


class AdaptiveAvgPool2dFunction(torch.autograd.Function):
    """Forward: one quantized mean per window.  Backward: every window's gradient spread evenly
    over the window, accumulated with a quantized add (mx/adaptive_avg_pooling.py:49-128).  Outputs
    are fp32 tensors, as in the reference."""

    @staticmethod
    def forward(ctx, input, output_size, mx_specs=None, name=None):
        B, C, H, W = input.size()
        oH, oW = _resolve_output_size(output_size, H, W)
        if input.dim() != 4:
            raise ValueError('expected 4D input (got {}D input)'.format(input.dim()))
        output = torch.zeros(B, C, oH, oW, device=input.device)
        for oh, h0, h1 in _windows(oH, H):
            for ow, w0, w1 in _windows(oW, W):
                output[:, :, oh, ow] = vec_reduce_mean(input[:, :, h0:h1, w0:w1], [2, 3], keepdim=False,
                                                       mx_specs=mx_specs)
        ctx.sizes = (B, C, H, W, oH, oW)
        ctx.device = input.device
        ctx.mx_specs = get_backwards_mx_specs(mx_specs)
        return output

    @staticmethod
    def backward(ctx, grad_output):
        B, C, H, W, oH, oW = ctx.sizes
        grad_input = torch.zeros(B, C, H, W, device=ctx.device)
        for oh, h0, h1 in _windows(oH, H):
            for ow, w0, w1 in _windows(oW, W):
                share = grad_output[:, :, oh, ow] / (h1 - h0) / (w1 - w0)
                share = share.view(B, C, 1, 1).expand(B, C, h1 - h0, w1 - w0)
                grad_input[:, :, h0:h1, w0:w1] = vec_add(grad_input[:, :, h0:h1, w0:w1], share,
                                                         mx_specs=ctx.mx_specs)
        return (grad_input, None, None, None)


def adaptive_avg_pool2d(input, output_size, mx_specs=None, name=None):
    mx_assert_test(mx_specs)
    if mx_specs is None:
        return f_adaptive_avg_pool2d(input, output_size)
    return AdaptiveAvgPool2dFunction.apply(input, output_size, apply_mx_specs(mx_specs), name)


class AdaptiveAvgPool2d(nn.Module):
    def __init__(self, output_size, mx_specs=None, name=None):
        super().__init__()
        mx_assert_test(mx_specs)
        self.mx_none = mx_specs is None
        self.output_size = output_size
        self.mx_specs = apply_mx_specs(mx_specs)
        self.name = name

    def forward(self, inputs):
        if self.mx_none:
            return f_adaptive_avg_pool2d(inputs, self.output_size)
        return AdaptiveAvgPool2dFunction.apply(inputs, self.output_size, self.mx_specs, self.name)
