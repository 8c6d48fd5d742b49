"""Elementwise (bfloat / fp) quantization: the call surface of the reference's mx/elemwise_ops.py,
served by the native kernels for every supported tensor.

Differences from the reference, on purpose:
  * there is one implementation per device -- HIP kernels for GPU tensors, the host library for CPU
    tensors -- and its results are bit-identical to the reference's pure-PyTorch path, so the
    ``custom_cuda`` switch is accepted but does not change the result;
  * ``round='dither'`` (stochastic, mx/elemwise_ops.py:57-59) runs natively too: the noise is drawn
    with torch.rand_like, as the reference does, and handed to the kernel; the kernels that run a
    whole chain of steps do not take it (those layers run their separate steps).
"""
import torch

from .formats import ROUNDING_VALUES, RoundingMode, _get_format_params, _get_max_norm


def _native_round(round):
    value = ROUNDING_VALUES.get(round) if type(round) is str else None
    if value is None:
        raise NotImplementedError(
            "rounding mode %r is not implemented by the native kernels (supported: %s)"
            % (round, ", ".join(RoundingMode.string_enums())))
    return value


def _quantize_elemwise_core(A, bits, exp_bits, max_norm, round='nearest',
                            saturate_normals=False, allow_denorm=True, custom_cuda=False):
    """Round every element of A to a format with `bits` = sign + implicit one + fraction bits and
    `exp_bits` exponent bits (0 = integer), overflowing to +-Inf or, if `saturate_normals`,
    clamping to +-max_norm.  Same contract as mx/elemwise_ops.py:82-170."""
    rmode = None if round == "dither" else _native_round(round)
    if A.is_sparse:
        if A.layout != torch.sparse_coo:
            raise NotImplementedError("Only COO layout sparse tensors are currently supported.")
        sp = A.coalesce()
        vals = _quantize_elemwise_core(sp.values().clone(), bits, exp_bits, max_norm, round=round,
                                       saturate_normals=saturate_normals,
                                       allow_denorm=allow_denorm, custom_cuda=custom_cuda)
        return torch.sparse_coo_tensor(sp.indices(), vals, sp.size(), dtype=sp.dtype,
                                       device=sp.device, requires_grad=sp.requires_grad)

    from . import custom_extensions
    if not A.is_contiguous() and A.dim() >= 2 and A.transpose(-1, -2).is_contiguous():
        # elementwise work does not care about the order of the axes: keep a transposed view
        # transposed (a K-major operand of the fused GEMM stays K-major) instead of copying it
        return _quantize_elemwise_core(A.transpose(-1, -2), bits, exp_bits, max_norm, round=round,
                                       saturate_normals=saturate_normals, allow_denorm=allow_denorm,
                                       custom_cuda=custom_cuda).transpose(-1, -2)
    A = A.contiguous()
    if round == "dither":
        # stochastic rounding: the noise comes from torch's generator, as in the reference
        # (torch.rand_like, mx/elemwise_ops.py:58), so torch.manual_seed governs it
        if A.device.type not in ("cuda", "cpu"):
            raise ValueError("Unrecognized device type %s" % A.device.type)
        return custom_extensions.funcs.quantize_elemwise_dither_func(
            A, torch.rand_like(A, requires_grad=False), bits, exp_bits, max_norm, saturate_normals, allow_denorm)
    if A.device.type == "cuda":
        return custom_extensions.funcs.quantize_elemwise_func_cuda(
            A, bits, exp_bits, max_norm, rmode, saturate_normals, allow_denorm)
    if A.device.type == "cpu":
        return custom_extensions.funcs.quantize_elemwise_func_cpp(
            A, bits, exp_bits, max_norm, rmode, saturate_normals, allow_denorm)
    raise ValueError("Unrecognized device type %s" % A.device.type)


def _quantize_elemwise(A, elem_format, round='nearest', custom_cuda=False,
                       saturate_normals=False, allow_denorm=True):
    """Quantize to a named element format (mx/elemwise_ops.py:173-188)."""
    if elem_format is None:
        return A
    ebits, mbits, _, max_norm, _ = _get_format_params(elem_format)
    return _quantize_elemwise_core(A, mbits, ebits, max_norm, round=round,
                                   allow_denorm=allow_denorm, saturate_normals=saturate_normals,
                                   custom_cuda=custom_cuda)


def _quantize_bfloat(A, bfloat, round='nearest', custom_cuda=False, allow_denorm=True):
    """bfloatX = 1 sign + 8 exponent + (X - 9) fraction bits (mx/elemwise_ops.py:191-206)."""
    if bfloat == 0 or bfloat == 32:
        return A
    return _quantize_elemwise_core(A, bits=bfloat - 7, exp_bits=8,
                                   max_norm=_get_max_norm(8, bfloat - 7), round=round,
                                   allow_denorm=allow_denorm, custom_cuda=custom_cuda)


def _quantize_fp(A, exp_bits=None, mantissa_bits=None, round='nearest', custom_cuda=False,
                 allow_denorm=True):
    """IEEE-style fpX with Inf/NaN in the top exponent (mx/elemwise_ops.py:209-230)."""
    if exp_bits is None or mantissa_bits is None:
        return A
    return _quantize_elemwise_core(A, bits=mantissa_bits + 2, exp_bits=exp_bits,
                                   max_norm=_get_max_norm(exp_bits, mantissa_bits + 2),
                                   round=round, allow_denorm=allow_denorm, custom_cuda=custom_cuda)


def elemwise_plan(mx_specs, round=None):
    """What quantize_elemwise_op(., mx_specs, round) amounts to, without a tensor:
    ("identity",), ("to_bf16",) or ("quantize", bits, exp_bits, max_norm, allow_denorm).  Raises the
    same ValueErrors.  Used by fused kernels that apply the quantizer between their own steps."""
    if mx_specs is None:
        return ("identity",)
    if round is None:
        round = mx_specs['round']
    if mx_specs['bfloat'] == 16 and round == 'even' and torch.cuda.is_bf16_supported() \
            and mx_specs['bfloat_subnorms'] == True:
        return ("to_bf16",)
    if mx_specs['bfloat'] > 0 and mx_specs['fp'] > 0:
        raise ValueError("Cannot set both [bfloat] and [fp] in mx_specs.")
    if mx_specs['bfloat'] > 9:
        b = mx_specs['bfloat']
        if b == 32:
            return ("identity",)
        return ("quantize", b - 7, 8, _get_max_norm(8, b - 7), bool(mx_specs['bfloat_subnorms']))
    if mx_specs['bfloat'] > 0:
        raise ValueError("Cannot set [bfloat] <= 9 in mx_specs.")
    if mx_specs['fp'] > 6:
        m = mx_specs['fp'] - 6
        return ("quantize", m + 2, 5, _get_max_norm(5, m + 2), bool(mx_specs['bfloat_subnorms']))
    if mx_specs['fp'] > 0:
        raise ValueError("Cannot set [fp] <= 6 in mx_specs.")
    return ("identity",)


_CHAIN_DTYPE_CODE = {torch.float32: 0, torch.bfloat16: 2}


def fused_chain_args(x, mx_specs, round=None):
    """For the kernels that run a whole chain of "tensor op, then quantize_elemwise_op" steps on a
    GPU tensor: (x, dtype code, (bits, exp_bits, max_norm, rounding code, allow_denorm)) with x
    cast to bf16 where the chain's first quantization would do that, or None when such a kernel
    cannot stand in for the chain (CPU or fp16 tensors, fused kernels switched off,
    round-half-even to a wide format on a bf16 tensor).  bits == 0 means "no format"."""
    from . import gemm
    if not (gemm.fused_enabled() and x.is_cuda):
        return None
    rnd = mx_specs['round'] if round is None else round
    if rnd == "dither":                  # needs a noise tensor per step: the separate steps draw it
        return None
    plan = elemwise_plan(mx_specs, rnd)
    if plan[0] == "to_bf16":
        x = x.to(torch.bfloat16)
        plan = ("identity",)
    if x.dtype not in _CHAIN_DTYPE_CODE:
        return None
    if plan[0] == "identity":
        return x, _CHAIN_DTYPE_CODE[x.dtype], (0, 0, 1.0, 0, 1)
    _, bits, exp_bits, max_norm, denorm = plan
    if x.dtype == torch.bfloat16 and bits >= 9 and rnd == 'even':
        return None
    return x, _CHAIN_DTYPE_CODE[x.dtype], (bits, exp_bits, max_norm, _native_round(rnd), int(denorm))


def quantize_elemwise_op(A, mx_specs, round=None):
    """Elementwise quantization selected by mx_specs['bfloat'] / ['fp']
    (mx/elemwise_ops.py:233-267)."""
    if mx_specs is None:
        return A
    if round is None:
        round = mx_specs['round']

    # torch's own cast is round-to-nearest-even to bfloat16; note it also changes the dtype
    if mx_specs['bfloat'] == 16 and round == 'even' and torch.cuda.is_bf16_supported() \
            and mx_specs['bfloat_subnorms'] == True:
        return A.to(torch.bfloat16)

    if mx_specs['bfloat'] > 0 and mx_specs['fp'] > 0:
        raise ValueError("Cannot set both [bfloat] and [fp] in mx_specs.")
    if mx_specs['bfloat'] > 9:
        return _quantize_bfloat(A, bfloat=mx_specs['bfloat'], round=round,
                                custom_cuda=mx_specs['custom_cuda'],
                                allow_denorm=mx_specs['bfloat_subnorms'])
    if mx_specs['bfloat'] > 0:
        raise ValueError("Cannot set [bfloat] <= 9 in mx_specs.")
    if mx_specs['fp'] > 6:
        return _quantize_fp(A, exp_bits=5, mantissa_bits=mx_specs['fp'] - 6, round=round,
                            custom_cuda=mx_specs['custom_cuda'],
                            allow_denorm=mx_specs['bfloat_subnorms'])
    if mx_specs['fp'] > 0:
        raise ValueError("Cannot set [fp] <= 6 in mx_specs.")
    return A
