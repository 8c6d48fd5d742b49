"""MX matmul: same interface as the reference's mx/matmul.py."""
import numpy as np
import torch

from .elemwise_ops import quantize_elemwise_op
from .gemm import inputs_can_skip_bfloat16_pass, mx_grad_contract, mx_matmul_contract
from .mx_ops import quantize_mx_op
from .specs import apply_mx_specs, get_backwards_mx_specs, mx_assert_test

torch_matmul = torch.matmul
torch_addmm = torch.addmm


def _fmt(specs, which, suffix=""):
    return specs[("a" if which == "a" else "w") + "_elem_format" + suffix]


class MatMulFunction(torch.autograd.Function):
    """in1 (..., M, K) x in2 (..., K, N) (+ bias).  `mode_config` says which spec ('a'ctivation or
    'w'eight format) each operand uses (mx/matmul.py:32-99; backward 101-200)."""

    @staticmethod
    def forward(ctx, in1, in2, bias, mx_specs, name, mode_config='aa'):
        assert mode_config in ["aa", "aw", "wa"]
        ctx.mode_config = mode_config
        if bias is None and inputs_can_skip_bfloat16_pass(ctx.needs_input_grad[:2], (in1, in2), mx_specs,
                                                          mx_specs["round_output"]):
            # inference: nothing keeps the quantized operands, the pack kernels quantize them
            out, finished = mx_matmul_contract(in1, in2, _fmt(mx_specs, mode_config[0]),
                                               _fmt(mx_specs, mode_config[1]), mx_specs,
                                               mx_specs["round_mx_output"],
                                               out_round=mx_specs["round_output"], pre_bfloat16=True)
            if out is not None:
                if not finished:
                    out = quantize_elemwise_op(out, mx_specs=mx_specs, round=mx_specs["round_output"])
                ctx.bias_shape = None
                ctx.mx_specs = get_backwards_mx_specs(mx_specs)
                return out
        bf_in1 = quantize_elemwise_op(in1, mx_specs=mx_specs, round=mx_specs["round_output"])
        bf_in2 = quantize_elemwise_op(in2, mx_specs=mx_specs, round=mx_specs["round_output"])
        if bias is not None:
            bf_bias = quantize_elemwise_op(bias, mx_specs=mx_specs, round=mx_specs["round_weight"])
            ctx.bias_shape = list(bias.shape)
        else:
            bf_bias, ctx.bias_shape = None, None
        if mx_specs["quantize_backprop"]:
            ctx.save_for_backward(bf_in1, bf_in2)
        else:
            ctx.save_for_backward(in1, in2)

        out, finished = mx_matmul_contract(bf_in1, bf_in2, _fmt(mx_specs, mode_config[0]),
                                           _fmt(mx_specs, mode_config[1]), mx_specs,
                                           mx_specs["round_mx_output"],
                                           out_round=mx_specs["round_output"], bias=bf_bias)
        if not finished:
            out = quantize_elemwise_op(out, mx_specs=mx_specs, round=mx_specs["round_output"])
            if bias is not None:
                out = quantize_elemwise_op(out + bf_bias, mx_specs=mx_specs,
                                           round=mx_specs["round_output"])
        ctx.mx_specs = get_backwards_mx_specs(mx_specs)
        return out

    @staticmethod
    def backward(ctx, grad_out):
        specs = ctx.mx_specs
        fmt1 = _fmt(specs, ctx.mode_config[0], "_bp")
        fmt2 = _fmt(specs, ctx.mode_config[1], "_bp")
        fmt_g = specs["a_elem_format_bp_os"]
        in1, in2 = ctx.saved_tensors
        grad_out = quantize_elemwise_op(grad_out, mx_specs=specs, round=specs["round_grad_input"])

        r_in, r_g = specs["round_mx_input_grad_input"], specs["round_mx_grad_output_grad_input"]
        if in1.dim() == in2.dim() and in1.shape[:-2] == in2.shape[:-2]:
            # grad_in1 = grad_out x in2^T over N (both along -1); grad_in2 = in1^T x grad_out over M
            # (both along -2)
            batched = in1.dim() == 3
            grad_in1 = mx_grad_contract(grad_out, fmt_g, r_g, False, in2, fmt2, r_in, False, specs,
                                        batched=batched)
            grad_in2 = mx_grad_contract(in1, fmt1, r_in, True, grad_out, fmt_g, r_g, True, specs,
                                        batched=batched)
        else:                                    # broadcast leading axes: torch.matmul sorts them out
            q1 = quantize_mx_op(in1, specs, elem_format=fmt1, axes=[-2], round=r_in)
            q2 = quantize_mx_op(in2, specs, elem_format=fmt2, axes=[-1], round=r_in)
            g_cols = quantize_mx_op(grad_out, specs, elem_format=fmt_g, axes=[-1], round=r_g)
            g_rows = quantize_mx_op(grad_out, specs, elem_format=fmt_g, axes=[-2], round=r_g)
            grad_in1 = torch_matmul(g_cols, q2.transpose(-1, -2))
            grad_in2 = torch_matmul(q1.transpose(-1, -2), g_rows)
        grad_in1 = quantize_elemwise_op(grad_in1, mx_specs=specs, round=specs["round_grad_input"])
        grad_in2 = quantize_elemwise_op(grad_in2, mx_specs=specs, round=specs["round_grad_input"])

        grad_bias = None
        if ctx.bias_shape is not None:
            inner = grad_out.shape[-1]
            assert np.prod(ctx.bias_shape) == inner
            grad_bias = grad_out.reshape(-1, inner).sum(0).reshape(ctx.bias_shape)
            grad_bias = quantize_elemwise_op(grad_bias, mx_specs=specs,
                                             round=specs["round_grad_weight"])
        return (grad_in1, grad_in2, grad_bias, None, None, None)


def matmul(in1, in2, bias=None, mx_specs=None, name=None, mode_config='aa'):
    mx_assert_test(mx_specs)
    if mx_specs is None:
        return torch_matmul(in1, in2) if bias is None else torch_addmm(bias, in1, in2)
    mx_specs = apply_mx_specs(mx_specs)
    return MatMulFunction.apply(in1, in2, bias, mx_specs, name, mode_config)
