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

_use_fused = True


def set_fused(enabled):
    """Globally allow (default) or forbid the fused packed-quantize + scaled-MFMA path."""
    global _use_fused
    _use_fused = bool(enabled)


def fused_enabled():
    return _use_fused


def _try_fused(a, b_kmajor, a_fmt, b_fmt, mx_specs, round, bias=None):
    """a: (..., M, K); b_kmajor: (..., N, K) -- both contiguous along K.  Returns None when the
    fused path does not apply."""
    if not _use_fused or not a.is_cuda:
        return None
    from . import fused
    return fused.mx_gemm_nt(a, b_kmajor, a_fmt, b_fmt, mx_specs, round, bias=bias)


def mx_linear_contract(x, w, a_fmt, w_fmt, mx_specs, round, fuse_bias=None):
    """x (..., K) times w (N, K) transposed: both operands share exponents along their last axis.
    fuse_bias: a bias the caller would add right after the product with no quantization step in
    between; returns (out, bias_was_added)."""
    out = _try_fused(x, w, a_fmt, w_fmt, mx_specs, round, bias=fuse_bias)
    if out is not None:
        return out, fuse_bias is not None
    qx = quantize_mx_op(x, mx_specs, elem_format=a_fmt, axes=[-1], round=round)
    qw = quantize_mx_op(w, mx_specs, elem_format=w_fmt, axes=[-1], round=round)
    # prequantized bf16 weights meet inputs of another dtype (mx/linear.py:77-80)
    if qw.dtype == torch.bfloat16 and qx.dtype != torch.bfloat16:
        qw = qw.to(qx.dtype)
    return torch.nn.functional.linear(qx, qw), False


def mx_matmul_contract(a, b, a_fmt, b_fmt, mx_specs, round, batched=False):
    """a (..., M, K) times b (..., K, N): a shares exponents along -1, b along -2."""
    if b.dim() >= 2 and a.dim() >= 2:
        # the fused kernel wants both operands K-major; a transposed view of b often already is
        bt = b.transpose(-1, -2)
        if bt.is_contiguous() and a.is_contiguous():
            out = _try_fused(a, bt, a_fmt, b_fmt, mx_specs, round)
            if out is not None:
                return out
    qa = quantize_mx_op(a, mx_specs, elem_format=a_fmt, axes=[-1], round=round)
    qb = quantize_mx_op(b, mx_specs, elem_format=b_fmt, axes=[-2], round=round)
    return torch.bmm(qa, qb) if batched else torch.matmul(qa, qb)
