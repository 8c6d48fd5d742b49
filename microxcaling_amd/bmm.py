"""MX batched matmul: same interface as the reference's mx/bmm.py."""
import torch

from .elemwise_ops import quantize_elemwise_op
from .gemm import inputs_can_skip_bfloat16_pass, mx_grad_contract, mx_matmul_contract
from .mx_ops import quantize_mx_op
from .specs import apply_mx_specs, get_backwards_mx_specs, mx_assert_test

torch_bmm = torch.bmm


class BMMFunction(torch.autograd.Function):
    """in1 (B, M, K) x in2 (B, K, N), both in the activation format (mx/bmm.py:20-67; backward
    69-127)."""

    @staticmethod
    def forward(ctx, in1, in2, mx_specs, name):
        if inputs_can_skip_bfloat16_pass(ctx.needs_input_grad[:2], (in1, in2), mx_specs,
                                         mx_specs["round_output"]):
            # inference: nothing keeps the quantized operands, the pack kernels quantize them
            out, finished = mx_matmul_contract(in1, in2, mx_specs["a_elem_format"],
                                               mx_specs["a_elem_format"], mx_specs,
                                               mx_specs["round_mx_output"], batched=True,
                                               out_round=mx_specs["round_output"], pre_bfloat16=True)
            if out is not None:
                if not finished:
                    out = quantize_elemwise_op(out, mx_specs=mx_specs, round=mx_specs["round_output"])
                ctx.mx_specs = get_backwards_mx_specs(mx_specs)
                return out
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
        fmt, fmt_g = specs["a_elem_format_bp"], specs["a_elem_format_bp_os"]
        r_in, r_g = specs["round_mx_input_grad_input"], specs["round_mx_grad_output_grad_input"]
        # grad_in1 = grad_out x in2^T over N (both along -1); grad_in2 = in1^T x grad_out over M
        # (both along -2)
        grad_in1 = mx_grad_contract(grad_out, fmt_g, r_g, False, in2, fmt, r_in, False, specs, batched=True)
        grad_in2 = mx_grad_contract(in1, fmt, r_in, True, grad_out, fmt_g, r_g, True, specs, batched=True)
        grad_in1 = quantize_elemwise_op(grad_in1, mx_specs=specs, round=specs["round_grad_input"])
        grad_in2 = quantize_elemwise_op(grad_in2, mx_specs=specs, round=specs["round_grad_input"])
        return (grad_in1, grad_in2, None, None)


def bmm(in1, in2, mx_specs=None, name=None):
    mx_assert_test(mx_specs)
    if mx_specs is None:
        return torch_bmm(in1, in2)
    mx_specs = apply_mx_specs(mx_specs)
    return BMMFunction.apply(in1, in2, mx_specs, name)
