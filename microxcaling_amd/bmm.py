"""MX batched matmul: same interface as the reference's mx/bmm.py."""
import torch

from .elemwise_ops import quantize_elemwise_op
from .gemm import mx_matmul_contract
from .mx_ops import quantize_mx_op
from .specs import apply_mx_specs, get_backwards_mx_specs, mx_assert_test

torch_bmm = torch.bmm


class BMMFunction(torch.autograd.Function):
    """in1 (B, M, K) x in2 (B, K, N), both in the activation format (mx/bmm.py:20-67; backward
    69-127)."""

    @staticmethod
    def forward(ctx, in1, in2, mx_specs, name):
        bf_in1 = quantize_elemwise_op(in1, mx_specs=mx_specs, round=mx_specs["round_output"])
        bf_in2 = quantize_elemwise_op(in2, mx_specs=mx_specs, round=mx_specs["round_output"])
        if mx_specs["quantize_backprop"]:
            ctx.save_for_backward(bf_in1, bf_in2)
        else:
            ctx.save_for_backward(in1, in2)
        out, finished = mx_matmul_contract(bf_in1, bf_in2, mx_specs["a_elem_format"],
                                           mx_specs["a_elem_format"], mx_specs,
                                           mx_specs["round_mx_output"], batched=True,
                                           out_round=mx_specs["round_output"])
        if not finished:
            out = quantize_elemwise_op(out, mx_specs=mx_specs, round=mx_specs["round_output"])
        ctx.mx_specs = get_backwards_mx_specs(mx_specs)
        return out

    @staticmethod
    def backward(ctx, grad_out):
        specs = ctx.mx_specs
        in1, in2 = ctx.saved_tensors
        grad_out = quantize_elemwise_op(grad_out, mx_specs=specs, round=specs["round_grad_input"])
        q1 = quantize_mx_op(in1, specs, elem_format=specs["a_elem_format_bp"], axes=[-2],
                            round=specs["round_mx_input_grad_input"])
        q2 = quantize_mx_op(in2, specs, elem_format=specs["a_elem_format_bp"], axes=[-1],
                            round=specs["round_mx_input_grad_input"])
        g_cols = quantize_mx_op(grad_out, specs, elem_format=specs["a_elem_format_bp_os"],
                                axes=[-1], round=specs["round_mx_grad_output_grad_input"])
        g_rows = quantize_mx_op(grad_out, specs, elem_format=specs["a_elem_format_bp_os"],
                                axes=[-2], round=specs["round_mx_grad_output_grad_input"])
        grad_in1 = torch_bmm(g_cols, q2.transpose(-1, -2))
        grad_in2 = torch_bmm(q1.transpose(-1, -2), g_rows)
        grad_in1 = quantize_elemwise_op(grad_in1, mx_specs=specs, round=specs["round_grad_input"])
        grad_in2 = quantize_elemwise_op(grad_in2, mx_specs=specs, round=specs["round_grad_input"])
        return (grad_in1, grad_in2, None, None)


def bmm(in1, in2, mx_specs=None, name=None):
    mx_assert_test(mx_specs)
    if mx_specs is None:
        return torch_bmm(in1, in2)
    mx_specs = apply_mx_specs(mx_specs)
    return BMMFunction.apply(in1, in2, mx_specs, name)
