"""MX transposed 2-d convolution: same interface as the reference's mx/transpose_convolution.py
(zero padding mode)."""
import torch
import torch.nn.functional as F

from .convolution import conv_weight
from .elemwise_ops import quantize_elemwise_op
from .mx_ops import quantize_mx_op
from .specs import apply_mx_specs, get_backwards_mx_specs, mx_assert_test

f_conv_transpose2d = F.conv_transpose2d
torch_conv2d = torch.conv2d


class ConvTranspose2dFunction(torch.autograd.Function):
    """The weight of a transposed convolution is (in, out / groups, kH, kW): the contracted axis is
    its axis 0, the input's axis 1 (mx/transpose_convolution.py:19-98).  Backward (100-199):
    grad_weight is the weight gradient of the forward convolution with input and grad_output
    swapped; grad_input is a plain convolution of grad_output with the weight."""

    @staticmethod
    def forward(ctx, input, weight, bias=None, stride=1, padding=0, output_padding=0, groups=1,
                dilation=1, mx_specs=None, name=None):
        assert input.shape[1] % groups == 0
        ctx.has_bias = bias is not None
        ctx.conv_args = dict(stride=stride, padding=padding, dilation=dilation, groups=groups)
        s = mx_specs
        bf_in = quantize_elemwise_op(input, mx_specs=s, round=s["round_output"])
        bf_weight = quantize_elemwise_op(weight, mx_specs=s, round=s["round_weight"])
        bf_bias = None if bias is None else quantize_elemwise_op(bias, mx_specs=s, round=s["round_weight"])
        if s["quantize_backprop"]:
            ctx.save_for_backward(bf_in, bf_weight)
        else:
            ctx.save_for_backward(input, weight)
        q_in = quantize_mx_op(bf_in, s, elem_format=s["a_elem_format"], axes=[1])
        q_w = quantize_mx_op(bf_weight, s, elem_format=s["w_elem_format"], axes=[0])
        out = f_conv_transpose2d(q_in, q_w, bf_bias, stride, padding, output_padding, groups, dilation)
        ctx.mx_specs = get_backwards_mx_specs(s)
        return quantize_elemwise_op(out, mx_specs=s, round=s["round_output"])

    @staticmethod
    def backward(ctx, grad_output):
        assert grad_output.shape[1] % ctx.conv_args["groups"] == 0
        input, weight = ctx.saved_tensors
        s = ctx.mx_specs
        g = quantize_elemwise_op(grad_output, mx_specs=s, round=s["round_grad_input"])

        ex_in = quantize_mx_op(input, s, elem_format=s["a_elem_format"], axes=[0])
        ex_g = quantize_mx_op(g, s, elem_format=s["a_elem_format"], axes=[0])
        grad_weight = conv_weight(ex_g, weight.shape, ex_in, **ctx.conv_args)
        grad_weight = quantize_elemwise_op(grad_weight, mx_specs=s, round=s["round_grad_weight"])

        od_w = quantize_mx_op(weight, s, elem_format=s["w_elem_format"], axes=[1])
        od_g = quantize_mx_op(g, s, elem_format=s["a_elem_format"], axes=[1])
        grad_input = torch_conv2d(od_g, od_w, bias=None, **ctx.conv_args)
        grad_input = quantize_elemwise_op(grad_input, mx_specs=s, round=s["round_grad_input"])

        grad_bias = None
        if ctx.has_bias:
            grad_bias = quantize_elemwise_op(g.sum(dim=(3, 2, 0)), mx_specs=s, round=s["round_grad_weight"])
        return (grad_input, grad_weight, grad_bias) + (None,) * 9


class ConvTranspose2d(torch.nn.ConvTranspose2d):
    def __init__(self, in_channels, out_channels, kernel_size, stride=1, padding=0,
                 output_padding=0, dilation=1, groups=1, bias=True, mx_specs=None, name=None):
        mx_assert_test(mx_specs)
        self.mx_none = mx_specs is None
        self.name = name
        self.mx_specs = apply_mx_specs(mx_specs)
        super().__init__(in_channels, out_channels, kernel_size, stride=stride, padding=padding,
                         dilation=dilation, output_padding=output_padding, groups=groups, bias=bias)

    def apply_mx_specs(self, mx_specs):
        self.mx_none = mx_specs is None
        self.mx_specs = apply_mx_specs(mx_specs)

    def append_name(self, postfix):
        self.name += postfix

    def forward(self, inputs, output_size=None):
        if self.mx_none:
            return super().forward(inputs, output_size)
        try:
            output_padding = self._output_padding(inputs, output_size, self.stride, self.padding,
                                                  self.kernel_size, 2, self.dilation)
        except TypeError:                     # older torch: no num_spatial_dims argument
            output_padding = self._output_padding(inputs, output_size, self.stride, self.padding,
                                                  self.kernel_size, self.dilation)
        return ConvTranspose2dFunction.apply(inputs, self.weight, self.bias, self.stride, self.padding,
                                             output_padding, self.groups, self.dilation,
                                             self.mx_specs, self.name)
