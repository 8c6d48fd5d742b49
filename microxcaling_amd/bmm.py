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


def _scores_operands(in1, in2, specs):
    """(in1, in2 transposed back) when the one-launch product + softmax kernel can take these operands
    (see bmm_softmax), else None."""
    from .gemm import pack_can_quantize_first
    from .fused import SCORES_K, SCORES_MAX_N
    if in1.dim() < 2 or in2.dim() != in1.dim() or in1.shape[:-2] != in2.shape[:-2]:
        return None
    wants_grad = torch.is_grad_enabled() and (in1.requires_grad or in2.requires_grad)
    if wants_grad or not inputs_can_skip_bfloat16_pass((False, False), (in1, in2), specs, specs["round_output"]):
        return None
    if not pack_can_quantize_first(specs, specs["round"]) or specs["vec_use_exp2"] or specs["vec_use_recip"]:
        return None
    from . import fused
    if fused._as_format(specs["a_elem_format"]) not in fused._PACKABLE or specs["block_size"] != 32 or \
            specs["shared_exp_method"] != "max" or in1.dtype != torch.bfloat16 or in2.dtype != torch.bfloat16:
        return None
    K, N = in1.shape[-1], in2.shape[-1]
    if K != SCORES_K or in2.shape[-2] != K or N == 0 or N % 32 != 0 or N > SCORES_MAX_N or in1.shape[-2] == 0:
        return None
    bt = in2.transpose(-1, -2)
    if not (bt.is_contiguous() and in1.is_contiguous()):
        return None
    return in1, bt


class DeferredProduct(torch.Tensor):
    """What mx.bmm returns for attention-shaped inference operands: the product, not yet computed.
    mx.softmax over its last axis computes product and softmax in one kernel (the logits never go to
    memory); every other use -- any torch op, in place or not, indexing, printing, .cpu() -- first
    evaluates the product exactly as mx.bmm would have (the GEMM kernel, once) and then runs on that
    tensor, so the object behaves like the logits tensor in every respect but one: the operands must
    not be modified in place before the product has been used (that raises)."""

    # results of ops on it are ordinary tensors (no re-wrapping by torch's default __torch_function__)
    __torch_function__ = torch._C._disabled_torch_function_impl

    @staticmethod
    def __new__(cls, in1, in2, specs, name):
        shape = in1.shape[:-1] + (in2.shape[-1],)
        r = torch.Tensor._make_wrapper_subclass(cls, shape, dtype=in1.dtype, device=in1.device)
        r._operands = (in1, in2, in1._version, in2._version)
        r._specs, r._name, r._value = specs, name, None
        return r

    def pending(self):
        """The operands (in1, in2, specs) while the product has not been evaluated, else None."""
        if self._value is not None:
            return None
        in1, in2, v1, v2 = self._operands
        if in1._version != v1 or in2._version != v2:
            raise RuntimeError("an operand of mx.bmm was modified in place before the product was used; the product "
                               "is evaluated on first use (gemm.set_deferred_scores(False) evaluates it at once)")
        return in1, in2, self._specs

    def materialize(self):
        if self._value is None:
            in1, in2, specs = self.pending()
            self._value = BMMFunction.apply(in1, in2, specs, self._name)
            self._operands = None
        return self._value

    def data_ptr(self):
        # the native entry points take raw pointers: they get the evaluated product's
        return self.materialize().data_ptr()

    @classmethod
    def __torch_dispatch__(cls, func, types, args=(), kwargs=None):
        from torch.utils._pytree import tree_map
        plain = lambda t: t.materialize() if isinstance(t, DeferredProduct) else t
        return func(*tree_map(plain, args), **tree_map(plain, kwargs or {}))

    def __repr__(self):
        return "DeferredProduct(%s, %s)" % (list(self.shape), "pending" if self._value is None else "evaluated")


def evaluated(t):
    """t itself, or the evaluated product if t is a DeferredProduct."""
    return t.materialize() if isinstance(t, DeferredProduct) else t


def bmm(in1, in2, mx_specs=None, name=None):
    mx_assert_test(mx_specs)
    if mx_specs is None:
        return torch_bmm(in1, in2)
    mx_specs = apply_mx_specs(mx_specs)
    in1, in2 = evaluated(in1), evaluated(in2)
    from .gemm import deferred_scores_enabled
    if deferred_scores_enabled() and in1.is_cuda and _scores_operands(in1, in2, mx_specs) is not None:
        return DeferredProduct(in1, in2, mx_specs, name)
    return BMMFunction.apply(in1, in2, mx_specs, name)


def _scores_in_one_launch(in1, in2, specs):
    """softmax(bmm(in1, in2), dim=-1) by the one-launch kernel, or None."""
    ops = _scores_operands(in1, in2, specs)
    if ops is None:
        return None
    from . import fused
    return fused.mx_bmm_softmax(ops[0], ops[1], specs["a_elem_format"], specs, specs["round_mx_output"],
                                exp2=bool(specs.get("softmax_exp2", False)))


def softmax_of_deferred(product, dim, softmax_specs):
    """mx.softmax(product, dim) in one launch when `product` is still pending, dim is its last axis and
    the softmax is asked for under the specs the product was asked for; else None (the caller evaluates
    the product and runs the softmax kernel)."""
    if not isinstance(product, DeferredProduct) or dim not in (-1, product.dim() - 1):
        return None
    pending = product.pending()
    if pending is None:
        return None
    in1, in2, specs = pending
    keys = ("bfloat", "fp", "round", "round_output", "bfloat_subnorms", "softmax_exp2", "vec_use_exp2", "vec_use_recip",
            "quantize_backprop", "custom_cuda")
    if any(softmax_specs.get(k) != specs.get(k) for k in keys):
        return None
    return _scores_in_one_launch(in1, in2, specs)


def bmm_softmax(in1, in2, mx_specs=None, name=None):
    """softmax(bmm(in1, in2), dim=-1): attention scores.  Same result as calling mx.bmm and then
    mx.softmax (mx/bmm.py:132-138, mx/softmax.py:91-97), which is also what runs whenever the one-launch
    form does not apply.  That form -- the logits stay in registers between the product and the
    softmax -- takes bf16 GPU operands when no gradient is wanted, in1 (..., M, 128), in2 a transposed
    view of a contiguous (..., N, 128) tensor with N a multiple of 32 up to 2048, an 8-bit-code MX
    format with block size 32, and mx_specs['bfloat'] = 16 with round-half-away (the quantizer applied
    after the product and after every softmax step).  It agrees with the two separate kernels
    within one step of the bfloat16 quantizer's grid on a few percent of the elements (the hardware
    exponential and the order of the row sum).  mx.softmax(mx.bmm(in1, in2), dim=-1) reaches the same
    kernel through bmm's deferred product (DeferredProduct)."""
    from .softmax import softmax
    mx_assert_test(mx_specs)
    if mx_specs is None:
        return torch.softmax(torch_bmm(in1, in2), dim=-1)
    specs = apply_mx_specs(mx_specs)
    in1, in2 = evaluated(in1), evaluated(in2)
    if in1.is_cuda:
        out = _scores_in_one_launch(in1, in2, specs)
        if out is not None:
            return out
    return softmax(bmm(in1, in2, mx_specs=mx_specs, name=name), dim=-1, mx_specs=mx_specs)
