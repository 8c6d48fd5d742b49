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


def bmm_softmax(in1, in2, mx_specs=None, name=None):
    """softmax(bmm(in1, in2), dim=-1): attention scores.  Same result as calling mx.bmm and then
    mx.softmax (mx/bmm.py:132-138, mx/softmax.py:91-97), which is also what runs whenever the one-launch
    form does not apply.  That form -- the logits stay in registers between the product and the
    softmax -- takes bf16 GPU operands when no gradient is wanted, in1 (..., M, 128), in2 a transposed
    view of a contiguous (..., N, 128) tensor with N a multiple of 32 up to 2048, an 8-bit-code MX
    format with block size 32, and mx_specs['bfloat'] = 16 with round-half-away (the quantizer applied
    after the product and after every softmax step).  It agrees with the two separate kernels
    within their own tolerance against the CPU chain (exp within 1 ulp, order of the row sum)."""
    from .softmax import softmax
    mx_assert_test(mx_specs)
    if mx_specs is None:
        return torch.softmax(torch_bmm(in1, in2), dim=-1)
    specs = apply_mx_specs(mx_specs)
    from .gemm import pack_can_quantize_first
    wants_grad = torch.is_grad_enabled() and (in1.requires_grad or in2.requires_grad)
    if (not wants_grad and in1.dim() >= 2 and in2.dim() >= 2
            and inputs_can_skip_bfloat16_pass((False, False), (in1, in2), specs, specs["round_output"])
            and pack_can_quantize_first(specs, specs["round"])
            and not specs["vec_use_exp2"] and not specs["vec_use_recip"]):
        bt = in2.transpose(-1, -2)
        if bt.is_contiguous() and in1.is_contiguous():
            from . import fused
            out = fused.mx_bmm_softmax(in1, bt, specs["a_elem_format"], specs, specs["round_mx_output"],
                                       exp2=bool(specs.get("softmax_exp2", False)))
            if out is not None:
                return out
    return softmax(bmm(in1, in2, mx_specs=mx_specs, name=name), dim=-1, mx_specs=mx_specs)
