"""MX convolutions (1d / 2d / 3d): same interface as the reference's mx/convolution.py.  Both
operands share exponents along the channel axis (axis 1, the contracted one); the convolution
itself is torch's (MIOpen on the GPU)."""
import torch
from torch.nn import grad

from .elemwise_ops import quantize_elemwise_op
from .mx_ops import quantize_mx_op
from .specs import apply_mx_specs, get_backwards_mx_specs, mx_assert_test

f_conv1d = torch.nn.functional.conv1d
f_conv2d = torch.nn.functional.conv2d
f_conv3d = torch.nn.functional.conv3d

# per number of spatial axes: forward, gradient wrt input, gradient wrt weight
_CONV = {1: (f_conv1d, grad.conv1d_input, grad.conv1d_weight),
         2: (f_conv2d, grad.conv2d_input, grad.conv2d_weight),
         3: (f_conv3d, grad.conv3d_input, grad.conv3d_weight)}


def conv_weight(input, weight_shape, grad_output, stride=1, padding=0, dilation=1, groups=1):
    """Gradient of convNd with respect to the weight (mx/convolution.py:21-101; torch >= 1.13 has a
    correct nn.grad.convNd_weight, which is all this needs)."""
    spatial = input.ndim - 2
    if spatial not in _CONV:
        raise ValueError("conv_weight does not work with input with ndim=%d" % input.ndim)
    return _CONV[spatial][2](input, weight_shape, grad_output, stride=stride, padding=padding,
                             dilation=dilation, groups=groups)


class ConvFunction(torch.autograd.Function):
    """Forward: bfloat-quantize input / weight / bias, MX-quantize input and weight along the
    channel axis, convolve (bias inside), bfloat-quantize (mx/convolution.py:104-194).
    Backward: grad_weight from operands MX-quantized along the batch axis, grad_input from the
    weight along axis 0 and grad_output along axis 1 (196-287)."""

    @staticmethod
    def forward(ctx, input, weight, bias=None, stride=1, padding=0, dilation=1, groups=1,
                mx_specs=None, name=None):
        spatial = input.ndim - 2
        assert spatial in _CONV
        assert input.shape[1] % groups == 0
        ctx.has_bias = bias is not None
        ctx.conv_args = dict(stride=stride, padding=padding, dilation=dilation, groups=groups)
        ctx.spatial = spatial
        s = mx_specs
        bf_in = quantize_elemwise_op(input, mx_specs=s, round=s["round_output"])
        bf_weight = quantize_elemwise_op(weight, mx_specs=s, round=s["round_weight"])
        bf_bias = None if bias is None else quantize_elemwise_op(bias, mx_specs=s, round=s["round_weight"])
        if s["quantize_backprop"]:
            ctx.save_for_backward(bf_in, bf_weight)
        else:
            ctx.save_for_backward(input, weight)
        q_in = quantize_mx_op(bf_in, s, elem_format=s['a_elem_format'], axes=[1])
        q_w = quantize_mx_op(bf_weight, s, elem_format=s['w_elem_format'], axes=[1])
        out = _CONV[spatial][0](q_in, q_w, bf_bias, stride, padding, dilation, groups)
        ctx.mx_specs = get_backwards_mx_specs(s)
        return quantize_elemwise_op(out, mx_specs=s, round=s["round_output"])

    @staticmethod
    def backward(ctx, grad_output):
        assert grad_output.shape[1] % ctx.conv_args["groups"] == 0
        input, weight = ctx.saved_tensors
        s = ctx.mx_specs
        g = quantize_elemwise_op(grad_output, mx_specs=s, round=s["round_grad_input"])

        ex_in = quantize_mx_op(input, s, elem_format=s['a_elem_format'], axes=[0])
        ex_g = quantize_mx_op(g, s, elem_format=s['a_elem_format'], axes=[0])
        grad_weight = conv_weight(ex_in, weight.shape, ex_g, **ctx.conv_args)
        grad_weight = quantize_elemwise_op(grad_weight, mx_specs=s, round=s["round_grad_weight"])

        od_w = quantize_mx_op(weight, s, elem_format=s['w_elem_format'], axes=[0])
        od_g = quantize_mx_op(g, s, elem_format=s['a_elem_format'], axes=[1])
        grad_input = _CONV[ctx.spatial][1](input.shape, od_w, od_g, **ctx.conv_args)
        grad_input = quantize_elemwise_op(grad_input, mx_specs=s, round=s["round_grad_input"])

        grad_bias = None
        if ctx.has_bias:
            grad_bias = quantize_elemwise_op(g.sum([0] + list(range(2, g.ndim))), mx_specs=s,
                                             round=s["round_grad_weight"])
        return (grad_input, grad_weight, grad_bias, None, None, None, None, None, None)


def _functional(plain):
    def conv(input, weight, bias=None, stride=1, padding=0, dilation=1, groups=1, mx_specs=None,
             name=None):
        mx_assert_test(mx_specs)
        if mx_specs is None:
            return plain(input, weight, bias=bias, stride=stride, padding=padding, dilation=dilation,
                         groups=groups)
        return ConvFunction.apply(input, weight, bias, stride, padding, dilation, groups,
                                  apply_mx_specs(mx_specs), name)
    conv.__name__ = plain.__name__
    return conv


conv1d = _functional(f_conv1d)
conv2d = _functional(f_conv2d)
conv3d = _functional(f_conv3d)


def _module(torch_cls):
    def __init__(self, in_channels, out_channels, kernel_size, stride=1, padding=0, dilation=1,
                 groups=1, bias=True, mx_specs=None, name=None):
        mx_assert_test(mx_specs)
        self.mx_none = mx_specs is None
        self.name = name
        self.mx_specs = apply_mx_specs(mx_specs)
        torch_cls.__init__(self, in_channels, out_channels, kernel_size, stride=stride,
                           padding=padding, dilation=dilation, groups=groups, bias=bias)

    def set_specs(self, mx_specs):
        self.mx_none = mx_specs is None
        self.mx_specs = apply_mx_specs(mx_specs)

    def append_name(self, postfix):
        self.name += postfix

    def forward(self, inputs):
        if self.mx_none:
            return torch_cls._conv_forward(self, inputs, self.weight, self.bias)
        return ConvFunction.apply(inputs, self.weight, self.bias, self.stride, self.padding,
                                  self.dilation, self.groups, self.mx_specs, self.name)

    return type(torch_cls.__name__, (torch_cls,), {"__init__": __init__, "apply_mx_specs": set_specs,
                                                   "append_name": append_name, "forward": forward})


Conv1d = _module(torch.nn.Conv1d)
Conv2d = _module(torch.nn.Conv2d)
Conv3d = _module(torch.nn.Conv3d)
