"""bfloat activations: same names, arguments and op order as the reference's mx/activations.py
(sigmoid, tanh, relu, relu6, leaky_relu, silu, gelu and their Module forms).  Every step is a
vector op followed by the elementwise quantizer, so on GPU tensors every step is one HIP kernel
launch plus torch's pointwise op."""
import torch
import torch.nn.functional as F

from .specs import apply_mx_specs, get_backwards_mx_specs, mx_assert_test
from .vector_ops import (vec_add, vec_exp, vec_mul, vec_quantize, vec_recip, vec_sub, vec_tanh)

f_gelu = F.gelu
f_relu6 = F.relu6
f_leaky_relu = F.leaky_relu
f_silu = F.silu
torch_relu = torch.relu
torch_relu_ = torch.relu_
torch_sigmoid = torch.sigmoid
torch_tanh = torch.tanh

# bfloat16-exact coefficients of the GELU approximations (mx/activations.py:472-475, 527-531)
GELU_FIRST_ORDER = 1.703125       # ~1.702
GELU_CUBIC = 0.044677734          # ~0.044715
GELU_SCALE = 1.59375              # ~1.5958
GELU_SCALE_DERIV = 0.21386719     # ~3 * 0.044715 * 1.5958


ACT_SIGMOID, ACT_TANH, ACT_SILU, ACT_GELU_FIRST_ORDER, ACT_GELU = range(5)


def _fused_forward(input, act, mx_specs, want_aux=False, want_q=False):
    """The whole forward chain of one activation as a single kernel launch
    (mxq_activation_forward): (output, logistic factor or None, quantized input or None), or None
    when the kernel does not cover the case (see fused_chain_args)."""
    from . import _lib
    from .custom_extensions import _flags_value
    from .elemwise_ops import fused_chain_args
    args = fused_chain_args(input, mx_specs)
    if args is None or input.numel() == 0:
        return None
    x, code, (bits, exp_bits, max_norm, rmode, denorm) = args
    x = x.contiguous()
    out = torch.empty_like(x)
    aux = torch.empty_like(x) if want_aux else None
    q = torch.empty_like(x) if want_q else None
    lib = _lib.gpu()
    with torch.cuda.device(x.device):
        rc = lib.mxq_activation_forward(x.data_ptr(), out.data_ptr(),
                                        None if aux is None else aux.data_ptr(),
                                        None if q is None else q.data_ptr(), code, x.numel(), act,
                                        bits, exp_bits, max_norm, rmode, denorm,
                                        2 if mx_specs['vec_use_exp2'] else 0, _flags_value(),
                                        torch.cuda.current_stream(x.device).cuda_stream)
    _lib.check(rc, lib)
    return out, aux, q


def _fused_backward(grad_output, act, saved, aux, mx_specs):
    """The backward chain of one activation as a single kernel launch (mxq_activation_backward)
    from the tensors the forward pass saved, or None when the kernel does not cover the case."""
    from . import _lib
    from .custom_extensions import _flags_value
    from .elemwise_ops import fused_chain_args
    args = fused_chain_args(grad_output, mx_specs)
    if args is None or grad_output.numel() == 0:
        return None
    g, code, (bits, exp_bits, max_norm, rmode, denorm) = args
    others = [saved] + ([aux] if aux is not None else [])
    if any(t.dtype != g.dtype or t.shape != g.shape or t.device != g.device for t in others):
        return None
    g, saved = g.contiguous(), saved.contiguous()
    aux = None if aux is None else aux.contiguous()
    out = torch.empty_like(g)
    lib = _lib.gpu()
    with torch.cuda.device(g.device):
        rc = lib.mxq_activation_backward(g.data_ptr(), saved.data_ptr(),
                                         None if aux is None else aux.data_ptr(), out.data_ptr(),
                                         code, g.numel(), act, bits, exp_bits, max_norm, rmode, denorm,
                                         _flags_value(), torch.cuda.current_stream(g.device).cuda_stream)
    _lib.check(rc, lib)
    return out


def _logistic(x, specs):
    """1 / (1 + exp(-x)) as three quantized steps (mx/activations.py:245-249)."""
    return vec_recip(vec_add(vec_exp(-x, mx_specs=specs), 1., mx_specs=specs), mx_specs=specs)


def _finish_inplace(ctx, input, output, inplace):
    if not inplace:
        return output
    ctx.mark_dirty(input)
    input.copy_(output)
    return input


def _masked_grad(mask, grad_output):
    zero = torch.zeros([1], dtype=grad_output.dtype, device=grad_output.device)
    return torch.where(mask, grad_output, zero)


class SigmoidFunction(torch.autograd.Function):
    """mx/activations.py:237-267; derivative s (1 - s) from the saved output."""

    @staticmethod
    def forward(ctx, input, mx_specs=None, name=None):
        fused = _fused_forward(input, ACT_SIGMOID, mx_specs)
        out = fused[0] if fused else _logistic(vec_quantize(input, mx_specs=mx_specs), mx_specs)
        ctx.save_for_backward(out)
        ctx.mx_specs = get_backwards_mx_specs(mx_specs)
        return out

    @staticmethod
    def backward(ctx, grad_output):
        out, = ctx.saved_tensors
        s = ctx.mx_specs
        fused = _fused_backward(grad_output, ACT_SIGMOID, out, None, s)
        if fused is not None:
            return (fused, None, None)
        g = vec_quantize(grad_output, mx_specs=s)
        d = vec_mul(out, vec_sub(1, out, mx_specs=s), mx_specs=s)
        return (vec_mul(d, g, mx_specs=s), None, None)


class TanhFunction(torch.autograd.Function):
    """mx/activations.py:270-297; derivative 1 - tanh^2."""

    @staticmethod
    def forward(ctx, input, mx_specs=None, name=None):
        fused = _fused_forward(input, ACT_TANH, mx_specs)
        out = fused[0] if fused else vec_tanh(vec_quantize(input, mx_specs=mx_specs), mx_specs=mx_specs)
        ctx.save_for_backward(out)
        ctx.mx_specs = get_backwards_mx_specs(mx_specs)
        return out

    @staticmethod
    def backward(ctx, grad_output):
        out, = ctx.saved_tensors
        s = ctx.mx_specs
        fused = _fused_backward(grad_output, ACT_TANH, out, None, s)
        if fused is not None:
            return (fused, None, None)
        g = vec_quantize(grad_output, mx_specs=s)
        d = vec_sub(1, vec_mul(out, out, mx_specs=s), mx_specs=s)
        return (vec_mul(d, g, mx_specs=s), None, None)


class ReLUFunction(torch.autograd.Function):
    """mx/activations.py:300-338: clamp first, quantize after; the gradient is masked, then
    quantized."""

    @staticmethod
    def forward(ctx, input, inplace=False, mx_specs=None, name=None):
        if inplace:
            ctx.mark_dirty(input)
            input = torch_relu_(input)
            input.copy_(vec_quantize(input, mx_specs=mx_specs))
            out = input
        else:
            out = vec_quantize(torch_relu(input), mx_specs=mx_specs)
        ctx.save_for_backward(out > 0)
        ctx.mx_specs = get_backwards_mx_specs(mx_specs)
        return out

    @staticmethod
    def backward(ctx, grad_output):
        mask, = ctx.saved_tensors
        return (vec_quantize(_masked_grad(mask, grad_output), mx_specs=ctx.mx_specs), None, None, None)


class ReLU6Function(torch.autograd.Function):
    """mx/activations.py:341-380."""

    @staticmethod
    def forward(ctx, input, inplace=False, mx_specs=None, name=None):
        if inplace:
            ctx.mark_dirty(input)
            input = f_relu6(input, inplace=True)
            input.copy_(vec_quantize(input, mx_specs=mx_specs))
            out = input
        else:
            out = vec_quantize(f_relu6(input), mx_specs=mx_specs)
        ctx.save_for_backward(torch.logical_and(out > 0, out < 6))
        ctx.mx_specs = get_backwards_mx_specs(mx_specs)
        return out

    @staticmethod
    def backward(ctx, grad_output):
        mask, = ctx.saved_tensors
        return (vec_quantize(_masked_grad(mask, grad_output), mx_specs=ctx.mx_specs), None, None, None)


class LeakyReLUFunction(torch.autograd.Function):
    """mx/activations.py:383-415."""

    @staticmethod
    def forward(ctx, input, negative_slope=0.01, inplace=False, mx_specs=None, name=None):
        ctx.negative_slope = negative_slope
        q = vec_quantize(input, mx_specs=mx_specs)
        out = vec_quantize(f_leaky_relu(q, negative_slope=negative_slope), mx_specs=mx_specs)
        out = _finish_inplace(ctx, input, out, inplace)
        ctx.save_for_backward(out > 0)
        ctx.mx_specs = get_backwards_mx_specs(mx_specs)
        return out

    @staticmethod
    def backward(ctx, grad_output):
        mask, = ctx.saved_tensors
        g = vec_quantize(grad_output, mx_specs=ctx.mx_specs)
        g_neg = vec_mul(g, ctx.negative_slope, mx_specs=ctx.mx_specs)
        return (torch.where(mask, g, g_neg), None, None, None, None)


class SiLUFunction(torch.autograd.Function):
    """x * sigmoid(x); derivative sigmoid + y (1 - sigmoid)  (mx/activations.py:418-455)."""

    @staticmethod
    def forward(ctx, input, inplace=False, mx_specs=None, name=None):
        fused = _fused_forward(input, ACT_SILU, mx_specs, want_aux=True)
        if fused:
            out, sig, _ = fused
        else:
            q = vec_quantize(input, mx_specs=mx_specs)
            sig = _logistic(q, mx_specs)
            out = vec_mul(q, sig, mx_specs=mx_specs)
        out = _finish_inplace(ctx, input, out, inplace)
        ctx.save_for_backward(out, sig)
        ctx.mx_specs = get_backwards_mx_specs(mx_specs)
        return out

    @staticmethod
    def backward(ctx, grad_output):
        y, sig = ctx.saved_tensors
        s = ctx.mx_specs
        fused = _fused_backward(grad_output, ACT_SILU, y, sig, s)
        if fused is not None:
            return (fused, None, None, None)
        g = vec_quantize(grad_output, mx_specs=s)
        d = vec_add(sig, vec_mul(y, vec_sub(1., sig, mx_specs=s), mx_specs=s), mx_specs=s)
        return (vec_mul(d, g, mx_specs=s), None, None, None)


class GELUFunction(torch.autograd.Function):
    """x * sigmoid(y) with y = 1.702 x (first order) or 1.5958 (x + 0.044715 x^3), coefficients at
    bfloat16 precision (mx/activations.py:458-557)."""

    @staticmethod
    def forward(ctx, input, mx_specs=None, first_order_gelu=False, name=None):
        ctx.first_order_gelu = first_order_gelu
        s = mx_specs
        fused = _fused_forward(input, ACT_GELU_FIRST_ORDER if first_order_gelu else ACT_GELU, s,
                               want_aux=True, want_q=bool(s['quantize_backprop']))
        if fused:
            out, phi, q = fused
            ctx.save_for_backward(q if s['quantize_backprop'] else input, phi)
            ctx.mx_specs = get_backwards_mx_specs(s)
            return out
        q = vec_quantize(input, mx_specs=s)
        if first_order_gelu:
            y = vec_mul(GELU_FIRST_ORDER, q, mx_specs=s)
        else:
            cube = vec_mul(vec_mul(q, q, mx_specs=s), q, mx_specs=s)
            y = vec_add(vec_mul(GELU_CUBIC, cube, mx_specs=s), q, mx_specs=s)
            y = vec_mul(GELU_SCALE, y, mx_specs=s)
        phi = _logistic(y, s)
        ctx.save_for_backward(q if s['quantize_backprop'] else input, phi)
        ctx.mx_specs = get_backwards_mx_specs(s)
        return vec_mul(q, phi, mx_specs=s)

    @staticmethod
    def backward(ctx, grad_output):
        x, phi = ctx.saved_tensors
        s = ctx.mx_specs
        fused = _fused_backward(grad_output, ACT_GELU_FIRST_ORDER if ctx.first_order_gelu else ACT_GELU,
                                x, phi, s)
        if fused is not None:
            return (fused, None, None, None)
        g = vec_quantize(grad_output, mx_specs=s)
        dphi = vec_mul(phi, vec_sub(1, phi, mx_specs=s), mx_specs=s)       # sigmoid'(y)
        if ctx.first_order_gelu:
            dphi = vec_mul(GELU_FIRST_ORDER, dphi, mx_specs=s)
        else:
            dy = vec_mul(GELU_SCALE_DERIV, vec_mul(x, x, mx_specs=s), mx_specs=s)
            dy = vec_add(GELU_SCALE, dy, mx_specs=s)
            dphi = vec_mul(dy, dphi, mx_specs=s)
        d = vec_add(phi, vec_mul(x, dphi, mx_specs=s), mx_specs=s)
        return (vec_mul(d, g, mx_specs=s), None, None, None)


# ---- functional forms (mx/activations.py:26-103) -------------------------------------------------
def sigmoid(input, mx_specs=None, name=None):
    mx_assert_test(mx_specs)
    if mx_specs is None:
        return torch_sigmoid(input)
    return SigmoidFunction.apply(input, apply_mx_specs(mx_specs), name)


def tanh(input, mx_specs=None, name=None):
    mx_assert_test(mx_specs)
    if mx_specs is None:
        return torch_tanh(input)
    return TanhFunction.apply(input, apply_mx_specs(mx_specs), name)


def relu(input, inplace=False, mx_specs=None, name=None):
    mx_assert_test(mx_specs)
    if mx_specs is None:
        return torch_relu_(input) if inplace else torch_relu(input)
    return ReLUFunction.apply(input, inplace, apply_mx_specs(mx_specs), name)


def relu6(input, inplace=False, mx_specs=None, name=None):
    mx_assert_test(mx_specs)
    if mx_specs is None:
        return f_relu6(input, inplace=inplace)
    return ReLU6Function.apply(input, inplace, apply_mx_specs(mx_specs), name)


def leaky_relu(input, negative_slope=0.01, inplace=False, mx_specs=None, name=None):
    mx_assert_test(mx_specs)
    if mx_specs is None:
        return f_leaky_relu(input, negative_slope=negative_slope, inplace=inplace)
    return LeakyReLUFunction.apply(input, negative_slope, inplace, apply_mx_specs(mx_specs), name)


def silu(input, inplace=False, mx_specs=None, name=None):
    mx_assert_test(mx_specs)
    if mx_specs is None:
        return f_silu(input, inplace=inplace)
    return SiLUFunction.apply(input, inplace, apply_mx_specs(mx_specs), name)


def gelu(input, mx_specs=None, first_order_gelu=False, approximate=None, name=None):
    """`approximate` only mirrors torch's signature: without mx_specs the tanh form is used, with
    mx_specs the sigmoid forms above."""
    mx_assert_test(mx_specs)
    if mx_specs is None and not first_order_gelu:
        try:
            return f_gelu(input, approximate='tanh')
        except TypeError:
            return f_gelu(input)
    return GELUFunction.apply(input, apply_mx_specs(mx_specs), first_order_gelu, name)


# ---- Module forms (mx/activations.py:108-232) ----------------------------------------------------
def _module(torch_cls, fn):
    """A torch.nn activation module that routes through `fn` when it has mx_specs.  Constructor
    arguments other than mx_specs / name are torch's own (inplace, negative_slope)."""
    def __init__(self, *args, mx_specs=None, name=None, **kwargs):
        torch_cls.__init__(self, *args, **kwargs)
        mx_assert_test(mx_specs)
        self.mx_none = mx_specs is None
        self.mx_specs = apply_mx_specs(mx_specs)
        self.name = name

    def set_specs(self, mx_specs):
        self.mx_none = mx_specs is None
        self.mx_specs = apply_mx_specs(mx_specs)

    def append_name(self, postfix):
        self.name += postfix

    def forward(self, input):
        if self.mx_none:
            return torch_cls.forward(self, input)
        kw = {k: getattr(self, k) for k in ("inplace", "negative_slope") if hasattr(self, k)}
        return fn(input, mx_specs=self.mx_specs, name=self.name, **kw)

    return type(torch_cls.__name__, (torch_cls,), {"__init__": __init__, "apply_mx_specs": set_specs,
                                                   "append_name": append_name, "forward": forward})


Sigmoid = _module(torch.nn.Sigmoid, sigmoid)
Tanh = _module(torch.nn.Tanh, tanh)
ReLU = _module(torch.nn.ReLU, relu)
ReLU6 = _module(torch.nn.ReLU6, relu6)
LeakyReLU = _module(torch.nn.LeakyReLU, leaky_relu)
SiLU = _module(torch.nn.SiLU, silu)


class GELU(torch.nn.GELU):
    def __init__(self, mx_specs=None, first_order_gelu=False, approximate=None, name=None):
        mx_assert_test(mx_specs)
        self.mx_none = mx_specs is None
        self.name = name
        self.mx_specs = apply_mx_specs(mx_specs)
        self.first_order_gelu = first_order_gelu
        try:
            super().__init__(approximate='tanh')
        except TypeError:
            super().__init__()

    def apply_mx_specs(self, mx_specs):
        self.mx_none = mx_specs is None
        self.mx_specs = apply_mx_specs(mx_specs)

    def append_name(self, postfix):
        self.name += postfix

    def forward(self, input):
        if self.mx_none and not self.first_order_gelu:
            return super().forward(input)
        return gelu(input, mx_specs=self.mx_specs, first_order_gelu=self.first_order_gelu,
                    name=self.name)
