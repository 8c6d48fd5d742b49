"""The dense contraction behind every MX matmul-like layer: MX-quantize both operands along the
contraction axis, multiply with fp32 accumulation.

Two implementations give results within accumulation-order tolerance of each other:
  * quantize kernels + torch's GEMM on the fake-quantized tensors (what the reference does,
    mx/linear.py:62-86, mx/matmul.py:68-91, mx/bmm.py:40-59);
  * the fused path (microxcaling_amd.fused): element codes + E8M0 scales consumed directly by the
    gfx950 scaled-MFMA GEMM.  Taken automatically when the operands qualify, unless switched off
    with set_fused(False).
"""
import torch

from .mx_ops import quantize_mx_op

# the stock torch functions, taken now: inject_pyt_ops later rebinds the names in the torch
# namespace to the MX versions, which end up here
f_linear = torch.nn.functional.linear
torch_matmul = torch.matmul
torch_bmm = torch.bmm

_use_fused = True


def set_fused(enabled):
    """Globally allow (default) or forbid the fused packed-quantize + scaled-MFMA path."""
    global _use_fused
    _use_fused = bool(enabled)


def fused_enabled():
    return _use_fused


_defer_scores = True


def set_deferred_scores(enabled):
    """mx.bmm on attention-shaped inference operands returns its product unevaluated (bmm.DeferredProduct)
    so that an mx.softmax over the last axis right after it can run product and softmax as one kernel;
    anything else that touches the result evaluates the product first.  enabled=False: mx.bmm always
    evaluates at once."""
    global _defer_scores
    _defer_scores = bool(enabled)


def deferred_scores_enabled():
    return _use_fused and _defer_scores


def _epilogue_mode(mx_specs, round, dtype):
    """How the layers' "elementwise-quantize the product (, add the bias, quantize again)" can ride
    in the fused GEMM's epilogue: 0 = the quantizer is the identity (plain rounding to the tensor
    dtype), 1 = bfloat16 with round-half-away on a bf16 tensor (closed form in the kernel),
    None = neither, the caller runs the separate steps."""
    from .elemwise_ops import elemwise_plan
    from .formats import _get_max_norm
    plan = elemwise_plan(mx_specs, round)
    if plan[0] == "identity" or (plan[0] == "to_bf16" and dtype == torch.bfloat16):
        return 0                 # (a cast to bf16 of a bf16 tensor: the case of prequantized weights)
    if plan == ("quantize", 9, 8, _get_max_norm(8, 9), True) and round == "nearest" \
            and dtype == torch.bfloat16:
        return 1
    return None


def _try_fused(a, b_kmajor, a_fmt, b_fmt, mx_specs, round, out_round=None, bias=None, pre_bfloat16=False,
               packed_b=None):
    """a: (..., M, K); b_kmajor: (..., N, K) -- both contiguous along K.  Returns (out, finished):
    out is None when the fused path does not apply; finished says whether the output quantization
    with rounding `out_round` and the bias add have been done in the epilogue."""
    if not _use_fused or not a.is_cuda:
        return None, False
    from . import fused
    mode = _epilogue_mode(mx_specs, out_round, a.dtype) if out_round is not None else None
    if mode is not None and (bias is None or bias.dtype == a.dtype):
        out = fused.mx_gemm_nt(a, b_kmajor, a_fmt, b_fmt, mx_specs, round, bias=bias,
                               epilogue_quant=mode == 1, pre_bfloat16=pre_bfloat16, packed_b=packed_b)
        if out is not None:
            return out, True
    return fused.mx_gemm_nt(a, b_kmajor, a_fmt, b_fmt, mx_specs, round, pre_bfloat16=pre_bfloat16,
                            packed_b=packed_b), False


def mx_linear_contract(x, w, a_fmt, w_fmt, mx_specs, round, out_round=None, bias=None, pre_bfloat16=False,
                       packed_w=None):
    """x (..., K) times w (N, K) transposed: both operands share exponents along their last axis.
    out_round / bias: what the caller does next -- elementwise-quantize the product with that
    rounding, add the (already quantized) bias, quantize again.  Returns (out, finished); when
    finished, those steps have been done in the GEMM's epilogue.  pre_bfloat16 (one flag per operand):
    as for mx_matmul_contract.  packed_w: the weight's packed form kept by a layer with prequantized
    weights (fused.pack_weight); w itself may then be an empty placeholder of the right dtype."""
    out, finished = _try_fused(x, w, a_fmt, w_fmt, mx_specs, round, out_round, bias, pre_bfloat16, packed_w)
    if out is not None:
        return out, finished
    if packed_w is not None and w.numel() == 0:
        raise RuntimeError("this layer keeps its weight as packed MX codes only, which only the fused GEMM "
                           "reads: the input must be a GPU tensor of the weight's dtype with the fused path on")
    if pre_bfloat16:
        return None, False
    qx = quantize_mx_op(x, mx_specs, elem_format=a_fmt, axes=[-1], round=round)
    qw = quantize_mx_op(w, mx_specs, elem_format=w_fmt, axes=[-1], round=round)
    # prequantized bf16 weights meet inputs of another dtype (mx/linear.py:77-80)
    if qw.dtype == torch.bfloat16 and qx.dtype != torch.bfloat16:
        qw = qw.to(qx.dtype)
    return f_linear(qx, qw), False


def inputs_can_skip_bfloat16_pass(needs_grad, tensors, mx_specs, round):
    """May a layer leave its operands' elementwise quantization to the pack kernels of the fused GEMM?
    Only when nothing keeps the quantized operands (no gradient is wanted), they are bf16 GPU tensors
    and the quantizer is bfloat16 with round-half-away, the form those kernels know."""
    return (not any(needs_grad) and all(t.is_cuda and t.dtype == torch.bfloat16 for t in tensors)
            and pack_can_quantize_first(mx_specs, round))


def pack_can_quantize_first(mx_specs, round):
    """Is quantize_elemwise_op(., mx_specs, round) on a bf16 tensor the bfloat16 / round-half-away
    quantizer that the pack kernel can apply itself, and are the fused kernels in use?"""
    return _use_fused and _epilogue_mode(mx_specs, round, torch.bfloat16) == 1


def mx_matmul_contract(a, b, a_fmt, b_fmt, mx_specs, round, batched=False, out_round=None, bias=None,
                       pre_bfloat16=False):
    """a (..., M, K) times b (..., K, N): a shares exponents along -1, b along -2.  out_round / bias
    and the return value: as for mx_linear_contract.  pre_bfloat16: a and b have not been through
    the elementwise quantization yet (see inputs_can_skip_bfloat16_pass); only the fused path takes
    them so, (None, False) means the caller has to quantize them and call again."""
    if b.dim() >= 2 and a.dim() >= 2:
        # the fused kernel wants both operands K-major; a transposed view of b often already is
        bt = b.transpose(-1, -2)
        if bt.is_contiguous() and a.is_contiguous():
            out, finished = _try_fused(a, bt, a_fmt, b_fmt, mx_specs, round, out_round, bias, pre_bfloat16)
            if out is not None:
                return out, finished
    if pre_bfloat16:
        return None, False
    qa = quantize_mx_op(a, mx_specs, elem_format=a_fmt, axes=[-1], round=round)
    qb = quantize_mx_op(b, mx_specs, elem_format=b_fmt, axes=[-2], round=round)
    return (torch_bmm(qa, qb) if batched else torch_matmul(qa, qb)), False


def mx_grad_contract(a, a_fmt, a_round, a_transposed, b, b_fmt, b_round, b_transposed, mx_specs,
                     batched=False):
    """The contractions of the backward passes: rows(a) x rows(b)^T over a shared K axis, each
    operand either (..., rows, K) quantized along -1, or -- transposed -- (..., K, rows) quantized
    along -2 (mx/linear.py:124-173, mx/matmul.py:131-172, mx/bmm.py:82-121).  Fused path: packed
    codes (transposed while packing where needed) + the scaled-MFMA GEMM; otherwise the
    fake-quantize kernels + torch's GEMM."""
    if _use_fused and a.is_cuda:
        from . import fused
        out = fused.mx_gemm_operands(((a, a_fmt, a_round, a_transposed), (b, b_fmt, b_round, b_transposed)),
                                     mx_specs, a.dtype)
        if out is not None:
            return out
    qa = quantize_mx_op(a, mx_specs, elem_format=a_fmt, axes=[-2 if a_transposed else -1], round=a_round)
    qb = quantize_mx_op(b, mx_specs, elem_format=b_fmt, axes=[-2 if b_transposed else -1], round=b_round)
    if a_transposed:
        qa = qa.transpose(-1, -2)
    if not b_transposed:
        qb = qb.transpose(-1, -2)
    return torch_bmm(qa, qb) if batched else torch_matmul(qa, qb)
