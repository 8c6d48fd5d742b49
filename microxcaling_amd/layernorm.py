"""LayerNorm and RMSNorm over the last axis: same interface as the reference's mx/layernorm.py."""
import torch
import torch.nn.functional as F

from .norm_utils import (layer_norm_rows, layer_norm_rows_grad_input, rms_norm_rows,
                         rms_norm_rows_grad_input)
from .specs import apply_mx_specs, get_backwards_mx_specs, mx_assert_test
from .vector_ops import vec_mul, vec_quantize, vec_reduce_sum

torch_layer_norm = F.layer_norm


MAX_FUSED_ROW = 16384


def _fused_forward(x, bf_weight, bf_bias, eps, mx_specs, rms):
    """The forward chain, including the quantization of the input x, as one kernel launch
    (mxq_norm_lastdim); weight and bias are already quantized.  Returns (output, x_norm, row
    statistic) or None when the kernel does not cover the case (CPU tensors, rows longer than 16384
    or not a multiple of 16 bytes, fp16, mixed dtypes, vec_use_recip, round-half-even to a wide
    format on bf16 tensors)."""
    from . import _lib
    from .custom_extensions import _flags_value
    from .elemwise_ops import fused_chain_args
    if mx_specs['vec_use_recip']:
        return None
    args = fused_chain_args(x, mx_specs)
    if args is None:
        return None
    x, code, (bits, exp_bits, max_norm, rmode, denorm) = args
    if bf_weight.dtype != x.dtype or bf_bias.dtype != x.dtype:
        return None
    n = x.shape[-1]
    if n == 0 or n > MAX_FUSED_ROW or n % (16 // x.element_size()) != 0 or bf_weight.numel() != n:
        return None
    x = x.contiguous()
    w, b = bf_weight.contiguous(), bf_bias.contiguous()
    out, x_norm = torch.empty_like(x), torch.empty_like(x)
    stat = torch.empty(x.shape[:-1] + (1,), dtype=x.dtype, device=x.device)
    lib = _lib.gpu()
    with torch.cuda.device(x.device):
        rc = lib.mxq_norm_lastdim(x.data_ptr(), w.data_ptr(), b.data_ptr(), out.data_ptr(),
                                  x_norm.data_ptr(), stat.data_ptr(), code,
                                  x.numel() // n, n, float(eps), int(rms), bits, exp_bits, max_norm,
                                  rmode, denorm, _flags_value(),
                                  torch.cuda.current_stream(x.device).cuda_stream)
    _lib.check(rc, lib)
    return out, x_norm, stat


def _leading_axes(t):
    return list(range(t.ndim - 1))


def _fused_grad_input(grad_output, weight, x_norm, stat, mx_specs, rms):
    """The gradient with respect to the input as one kernel launch (mxq_norm_backward_lastdim) from
    the saved normalized input and row statistic, under the conditions of _fused_forward; None
    otherwise."""
    from . import _lib
    from .custom_extensions import _flags_value
    from .elemwise_ops import fused_chain_args
    if mx_specs['vec_use_recip']:
        return None
    args = fused_chain_args(grad_output, mx_specs)
    if args is None:
        return None
    g, code, (bits, exp_bits, max_norm, rmode, denorm) = args
    n = g.shape[-1]
    if n == 0 or n > MAX_FUSED_ROW or n % (16 // g.element_size()) != 0 or weight.numel() != n:
        return None
    rows = g.numel() // n
    if any(t.dtype != g.dtype or t.device != g.device for t in (weight, x_norm, stat)) \
            or x_norm.shape != g.shape or stat.numel() != rows:
        return None
    g, w, z, st = g.contiguous(), weight.contiguous(), x_norm.contiguous(), stat.contiguous()
    out = torch.empty_like(g)
    lib = _lib.gpu()
    with torch.cuda.device(g.device):
        rc = lib.mxq_norm_backward_lastdim(g.data_ptr(), w.data_ptr(), z.data_ptr(), st.data_ptr(),
                                           out.data_ptr(), code, rows, n, int(rms), bits, exp_bits,
                                           max_norm, rmode, denorm, _flags_value(),
                                           torch.cuda.current_stream(g.device).cuda_stream)
    _lib.check(rc, lib)
    return out


def _fused_param_grads(grad_output, x_norm, mx_specs):
    """(grad_weight, grad_bias) as two kernel launches that read grad_output and x_norm once
    (mxq_norm_param_grads), under the conditions of the other fused kernels; None otherwise."""
    from . import _lib
    from .custom_extensions import _flags_value
    from .elemwise_ops import fused_chain_args
    args = fused_chain_args(grad_output, mx_specs)
    if args is None:
        return None
    g, code, (bits, exp_bits, max_norm, rmode, denorm) = args
    n = g.shape[-1] if g.ndim else 0
    if g.ndim < 2 or n == 0 or n % (16 // g.element_size()) != 0:
        return None
    rows = g.numel() // n
    if rows == 0 or x_norm.dtype != g.dtype or x_norm.device != g.device or x_norm.shape != g.shape:
        return None
    g, z = g.contiguous(), x_norm.contiguous()
    grad_weight = torch.empty(n, dtype=g.dtype, device=g.device)
    grad_bias = torch.empty(n, dtype=g.dtype, device=g.device)
    lib = _lib.gpu()
    ws_bytes = lib.mxq_norm_param_grads_workspace_bytes(code, rows, n)
    ws = torch.empty(ws_bytes // 4, dtype=torch.float32, device=g.device)
    with torch.cuda.device(g.device):
        rc = lib.mxq_norm_param_grads(g.data_ptr(), z.data_ptr(), grad_weight.data_ptr(),
                                      grad_bias.data_ptr(), ws.data_ptr(), ws_bytes, code, rows, n,
                                      bits, exp_bits, max_norm, rmode, denorm, _flags_value(),
                                      torch.cuda.current_stream(g.device).cuda_stream)
    _lib.check(rc, lib)
    return grad_weight, grad_bias


def _fused_backward(grad_output, weight, x_norm, stat, mx_specs, rms):
    """(grad_input, grad_weight, grad_bias) from the output gradient as it arrives: both kernels
    quantize it on the way in, so the separate quantization pass is not run.  None unless both
    kernels cover the case."""
    from .elemwise_ops import fused_chain_args
    args = fused_chain_args(grad_output, mx_specs)
    if args is None:
        return None
    g = args[0]                          # cast to bf16 once where the quantization is that cast
    params = _fused_param_grads(g, x_norm, mx_specs)
    if params is None:
        return None
    grad_input = _fused_grad_input(g, weight, x_norm, stat, mx_specs, rms)
    if grad_input is None:
        return None
    return grad_input, params[0], params[1]


def _param_grads(grad_output, x_norm, specs):
    """grad_bias = sum(g), grad_weight = sum(g * x_norm) over every axis but the last."""
    fused = _fused_param_grads(grad_output, x_norm, specs)
    if fused is not None:
        return fused
    axes = _leading_axes(grad_output)
    grad_bias = vec_reduce_sum(grad_output, axes, mx_specs=specs)
    grad_weight = vec_reduce_sum(vec_mul(grad_output, x_norm, mx_specs=specs), axes, mx_specs=specs)
    return grad_weight, grad_bias


class LayerNormFunction(torch.autograd.Function):
    """mx/layernorm.py:17-69."""

    @staticmethod
    def forward(ctx, x, weight, bias, eps, mx_specs=None, name=None):
        ctx.eps = eps
        bf_weight = vec_quantize(weight, mx_specs=mx_specs)
        bf_bias = vec_quantize(bias, mx_specs=mx_specs)
        fused = _fused_forward(x, bf_weight, bf_bias, eps, mx_specs, rms=False)
        if fused is not None:
            output, x_norm, x_vare = fused
        else:
            output, x_norm, x_vare = layer_norm_rows(vec_quantize(x, mx_specs=mx_specs), bf_weight, bf_bias, eps,
                                                     mx_specs)
        ctx.save_for_backward(x_norm, x_vare, bf_weight if mx_specs['quantize_backprop'] else weight)
        ctx.mx_specs = get_backwards_mx_specs(mx_specs)
        return output

    @staticmethod
    def backward(ctx, grad_output):
        x_norm, x_vare, weight = ctx.saved_tensors
        s = ctx.mx_specs
        fused = _fused_backward(grad_output, weight, x_norm, x_vare, s, rms=False)
        if fused is not None:
            return fused + (None, None, None)
        grad_output = vec_quantize(grad_output, mx_specs=s)
        grad_weight, grad_bias = _param_grads(grad_output, x_norm, s)
        grad_input = _fused_grad_input(grad_output, weight, x_norm, x_vare, s, rms=False)
        if grad_input is None:
            grad_input = layer_norm_rows_grad_input(grad_output, weight, x_norm, x_vare, s)
        return (grad_input, grad_weight, grad_bias, None, None, None)


class RMSNormFunction(torch.autograd.Function):
    """x / sqrt(mean(x^2) + eps) * weight + bias (mx/layernorm.py:100-168)."""

    @staticmethod
    def forward(ctx, x, weight, bias, eps, mx_specs=None, name=None):
        ctx.eps = eps
        s = mx_specs
        bf_weight = vec_quantize(weight, mx_specs=s)
        bf_bias = vec_quantize(bias, mx_specs=s)
        fused = _fused_forward(x, bf_weight, bf_bias, eps, s, rms=True)
        if fused is not None:
            output, x_norm, rms_inv = fused
        else:
            output, x_norm, rms_inv = rms_norm_rows(vec_quantize(x, mx_specs=s), bf_weight, bf_bias, eps, s)
        ctx.save_for_backward(x_norm, rms_inv, bf_weight if s['quantize_backprop'] else weight)
        ctx.mx_specs = get_backwards_mx_specs(s)
        return output

    @staticmethod
    def backward(ctx, grad_output):
        x_norm, rms_inv, weight = ctx.saved_tensors
        s = ctx.mx_specs
        fused = _fused_backward(grad_output, weight, x_norm, rms_inv, s, rms=True)
        if fused is not None:
            return fused + (None, None, None)
        grad_output = vec_quantize(grad_output, mx_specs=s)
        grad_weight, grad_bias = _param_grads(grad_output, x_norm, s)
        fused = _fused_grad_input(grad_output, weight, x_norm, rms_inv, s, rms=True)
        if fused is not None:
            return (fused, grad_weight, grad_bias, None, None, None)
        grad_input = rms_norm_rows_grad_input(grad_output, weight, x_norm, rms_inv, s)
        return (grad_input, grad_weight, grad_bias, None, None, None)


class _NormModule(torch.nn.LayerNorm):
    """TF-style layer norm module (epsilon inside the square root)."""
    _function = None
    _plain_without_specs = True

    def __init__(self, hidden_size, eps=1e-12, mx_specs=None, name=None):
        mx_assert_test(mx_specs)
        self.mx_none = mx_specs is None
        self.name = name
        self.mx_specs = apply_mx_specs(mx_specs)
        super().__init__(normalized_shape=hidden_size, eps=eps)

    def apply_mx_specs(self, mx_specs):
        self.mx_none = mx_specs is None
        self.mx_specs = apply_mx_specs(mx_specs)

    def append_name(self, postfix):
        self.name += postfix

    def forward(self, x):
        if self.mx_none and self._plain_without_specs:
            return super().forward(x)
        return self._function.apply(x, self.weight, self.bias, self.eps, self.mx_specs, self.name)


class LayerNorm(_NormModule):
    _function = LayerNormFunction


class RMSNorm(_NormModule):
    """torch has no RMSNorm to fall back to: always the vector-op chain (mx/layernorm.py:171-196)."""
    _function = RMSNormFunction
    _plain_without_specs = False


def layer_norm(input, normalized_shape, weight, bias, eps=1e-12, mx_specs=None, name=None):
    mx_assert_test(mx_specs)
    if mx_specs is None:
        return torch_layer_norm(input, normalized_shape, weight, bias, eps)
    assert normalized_shape == weight.shape
    return LayerNormFunction.apply(input, weight, bias, eps, apply_mx_specs(mx_specs), name)
