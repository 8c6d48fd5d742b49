"""Differentiable elementwise and reduction ops with bfloat quantization after every step: same
names and behaviour as the reference's mx/simd_ops.py (simd_add / sub / mul / div / split / square /
sqrt / exp / log / reduce_sum / reduce_mean / norm).  Binary ops accept a tensor or a Python scalar
as second operand and broadcast like torch."""
import numpy as np
import torch

from .specs import apply_mx_specs, get_backwards_mx_specs, mx_assert_test
from .vector_ops import (vec_add, vec_div, vec_exp, vec_mul, vec_quantize, vec_reduce_sum, vec_sqrt,
                         vec_sub)

torch_sum = torch.sum
torch_mean = torch.mean
torch_sqrt = torch.sqrt
torch_exp = torch.exp
torch_log = torch.log
torch_square = torch.square


def _broadcast_gradient(grad_out, in_shape, mx_specs):
    """Gradient of broadcasting `in_shape` up to grad_out's shape: sum (quantized before and after)
    over the axes that were created or stretched (mx/simd_ops.py:41-79)."""
    if list(grad_out.shape) == in_shape:
        return grad_out
    assert grad_out.ndim >= len(in_shape)
    reduce_dims = []
    for i in range(grad_out.ndim):
        if i + 1 > len(in_shape):
            reduce_dims.append(-1 - i)
        elif grad_out.shape[-1 - i] != in_shape[-1 - i]:
            if in_shape[-1 - i] != 1:
                raise ValueError("simd gradient shape error: grad_out is %s and the input is %s"
                                 % (tuple(grad_out.shape), in_shape))
            reduce_dims.append(-1 - i)
    if not reduce_dims:
        return grad_out.view(in_shape)
    g = torch_sum(vec_quantize(grad_out, mx_specs=mx_specs), dim=reduce_dims)
    return vec_quantize(g, mx_specs=mx_specs).view(in_shape)


def _prepare_binary(ctx, in1, in2, mx_specs):
    """Quantize the tensor operands; remember shapes for the broadcast gradient.  Returns
    (q1, q2) with q2 the scalar itself when in2 is not a tensor."""
    assert isinstance(in1, torch.Tensor)
    ctx.mx_specs = get_backwards_mx_specs(mx_specs)
    q1 = vec_quantize(in1, mx_specs=mx_specs)
    ctx.in2_const = not isinstance(in2, torch.Tensor)
    if ctx.in2_const:
        ctx.in2 = in2
        return q1, in2
    ctx.in1_shape, ctx.in2_shape = list(in1.shape), list(in2.shape)
    return q1, vec_quantize(in2, mx_specs=mx_specs)


class SIMDAdd(torch.autograd.Function):
    @staticmethod
    def forward(ctx, in1, in2, mx_specs=None):
        q1, q2 = _prepare_binary(ctx, in1, in2, mx_specs)
        return vec_add(q1, q2, mx_specs=mx_specs)

    @staticmethod
    def backward(ctx, g):
        s = ctx.mx_specs
        g = vec_quantize(g, mx_specs=s)
        if ctx.in2_const:
            return (g, None, None)
        return (_broadcast_gradient(g, ctx.in1_shape, s), _broadcast_gradient(g, ctx.in2_shape, s), None)


class SIMDSub(torch.autograd.Function):
    @staticmethod
    def forward(ctx, in1, in2, mx_specs=None):
        q1, q2 = _prepare_binary(ctx, in1, in2, mx_specs)
        return vec_sub(q1, q2, mx_specs=mx_specs)

    @staticmethod
    def backward(ctx, g):
        s = ctx.mx_specs
        if ctx.in2_const:
            return (g, None, None)
        # only the negated gradient is quantized here (mx/simd_ops.py:139-146)
        neg = vec_quantize(-g, mx_specs=s)
        return (_broadcast_gradient(g, ctx.in1_shape, s), _broadcast_gradient(neg, ctx.in2_shape, s), None)


class SIMDMul(torch.autograd.Function):
    @staticmethod
    def forward(ctx, in1, in2, mx_specs=None):
        q1, q2 = _prepare_binary(ctx, in1, in2, mx_specs)
        keep_q = mx_specs['quantize_backprop']
        if ctx.in2_const:
            ctx.save_for_backward(q1 if keep_q else in1)
        else:
            ctx.save_for_backward(*((q1, q2) if keep_q else (in1, in2)))
        return vec_mul(q1, q2, mx_specs=mx_specs)

    @staticmethod
    def backward(ctx, g):
        s = ctx.mx_specs
        g = vec_quantize(g, mx_specs=s)
        if ctx.in2_const:
            return (vec_mul(g, ctx.in2, mx_specs=s), None, None)
        in1, in2 = ctx.saved_tensors
        g1 = _broadcast_gradient(vec_mul(g, in2, mx_specs=s), ctx.in1_shape, s)
        g2 = _broadcast_gradient(vec_mul(g, in1, mx_specs=s), ctx.in2_shape, s)
        return (g1, g2, None)


class SIMDDiv(torch.autograd.Function):
    """d/dx1 = 1 / x2, d/dx2 = -(x1 / x2) / x2 from the saved quotient."""

    @staticmethod
    def forward(ctx, in1, in2, mx_specs=None):
        q1, q2 = _prepare_binary(ctx, in1, in2, mx_specs)
        out = vec_div(q1, q2, mx_specs=mx_specs)
        keep_q = mx_specs['quantize_backprop']
        if ctx.in2_const:
            ctx.save_for_backward(q1 if keep_q else in1)
        else:
            ctx.save_for_backward(out, q2 if keep_q else in2)
        return out

    @staticmethod
    def backward(ctx, g):
        s = ctx.mx_specs
        g = vec_quantize(g, mx_specs=s)
        if ctx.in2_const:
            return (vec_div(g, ctx.in2, mx_specs=s), None, None)
        out, in2 = ctx.saved_tensors
        g1 = vec_div(g, in2, mx_specs=s)
        g2 = vec_mul(g, vec_div(-out, in2, mx_specs=s), mx_specs=s)
        return (_broadcast_gradient(g1, ctx.in1_shape, s), _broadcast_gradient(g2, ctx.in2_shape, s), None)


class SIMDSplit(torch.autograd.Function):
    """Two copies forward; the two gradients are added (quantized) backward."""

    @staticmethod
    def forward(ctx, in1, mx_specs=None):
        ctx.mx_specs = get_backwards_mx_specs(mx_specs)
        ctx.set_materialize_grads(False)
        return in1.clone(), in1.clone()

    @staticmethod
    def backward(ctx, g1, g2):
        if g1 is None:
            return (g2, None)
        if g2 is None:
            return (g1, None)
        s = ctx.mx_specs
        return (vec_add(vec_quantize(g1, mx_specs=s), vec_quantize(g2, mx_specs=s), mx_specs=s), None)


class SIMDSquare(torch.autograd.Function):
    @staticmethod
    def forward(ctx, in1, mx_specs=None):
        ctx.mx_specs = get_backwards_mx_specs(mx_specs)
        q = vec_quantize(in1, mx_specs=mx_specs)
        ctx.save_for_backward(q if mx_specs['quantize_backprop'] else in1)
        return vec_quantize(q ** 2, mx_specs=mx_specs)

    @staticmethod
    def backward(ctx, g):
        x, = ctx.saved_tensors
        s = ctx.mx_specs
        g = vec_quantize(g, mx_specs=s)
        return (vec_mul(g, vec_mul(x, 2, mx_specs=s), mx_specs=s), None)


class SIMDSqrt(torch.autograd.Function):
    @staticmethod
    def forward(ctx, in1, mx_specs=None):
        ctx.mx_specs = get_backwards_mx_specs(mx_specs)
        out = vec_sqrt(vec_quantize(in1, mx_specs=mx_specs), mx_specs=mx_specs)
        ctx.save_for_backward(out)
        return out

    @staticmethod
    def backward(ctx, g):
        root, = ctx.saved_tensors
        s = ctx.mx_specs
        g = vec_mul(vec_quantize(g, mx_specs=s), 0.5, mx_specs=s)
        return (vec_div(g, root, mx_specs=s), None)


class SIMDExp(torch.autograd.Function):
    @staticmethod
    def forward(ctx, in1, mx_specs=None):
        ctx.mx_specs = get_backwards_mx_specs(mx_specs)
        out = vec_exp(vec_quantize(in1, mx_specs=mx_specs), mx_specs=mx_specs)
        ctx.save_for_backward(out)
        return out

    @staticmethod
    def backward(ctx, g):
        out, = ctx.saved_tensors
        s = ctx.mx_specs
        return (vec_mul(vec_quantize(g, mx_specs=s), out, mx_specs=s), None)


class SIMDLog(torch.autograd.Function):
    @staticmethod
    def forward(ctx, in1, mx_specs=None):
        ctx.mx_specs = get_backwards_mx_specs(mx_specs)
        q = vec_quantize(in1, mx_specs=mx_specs)
        ctx.save_for_backward(q if mx_specs['quantize_backprop'] else in1)
        return vec_quantize(torch_log(q), mx_specs=mx_specs)

    @staticmethod
    def backward(ctx, g):
        x, = ctx.saved_tensors
        s = ctx.mx_specs
        return (vec_div(vec_quantize(g, mx_specs=s), x, mx_specs=s), None)


class SIMDReduceSum(torch.autograd.Function):
    @staticmethod
    def forward(ctx, in1, dim, keepdim=False, mx_specs=None):
        ctx.mx_specs = get_backwards_mx_specs(mx_specs)
        ctx.dim = [dim] if type(dim) == int else dim
        ctx.keepdim = keepdim
        ctx.input_shape = list(in1.shape)
        return vec_reduce_sum(vec_quantize(in1, mx_specs=mx_specs), ctx.dim, keepdim=keepdim,
                              mx_specs=mx_specs)

    @staticmethod
    def backward(ctx, g):
        ndim = len(ctx.input_shape)
        dims = [d + ndim if d < 0 else d for d in ctx.dim]
        g = vec_quantize(g, mx_specs=ctx.mx_specs)
        if not ctx.keepdim:
            for d in sorted(dims):
                g = g.unsqueeze(d)
        sizes = [ctx.input_shape[d] if d in dims else -1 for d in range(ndim)]
        return (g.expand(sizes), None, None, None)


def _unary(function, plain):
    def op(in1, mx_specs=None):
        mx_assert_test(mx_specs)
        if mx_specs is None:
            return plain(in1)
        return function.apply(in1, apply_mx_specs(mx_specs))
    return op


def _binary(function, plain):
    def op(in1, in2, mx_specs=None):
        mx_assert_test(mx_specs)
        if mx_specs is None:
            return plain(in1, in2)
        return function.apply(in1, in2, apply_mx_specs(mx_specs))
    return op


simd_add = _binary(SIMDAdd, lambda a, b: a + b)
simd_sub = _binary(SIMDSub, lambda a, b: a - b)
simd_mul = _binary(SIMDMul, lambda a, b: a * b)
simd_div = _binary(SIMDDiv, lambda a, b: a / b)
simd_split = _unary(SIMDSplit, lambda a: (a, a))
simd_square = _unary(SIMDSquare, torch_square)
simd_sqrt = _unary(SIMDSqrt, torch_sqrt)
simd_exp = _unary(SIMDExp, torch_exp)
simd_log = _unary(SIMDLog, torch_log)


def simd_reduce_sum(in1, dim=None, keepdim=False, mx_specs=None):
    mx_assert_test(mx_specs)
    if dim is None:
        dim = list(range(in1.ndim))
    if mx_specs is None:
        return torch_sum(in1, dim, keepdim=keepdim)
    return SIMDReduceSum.apply(in1, dim, keepdim, apply_mx_specs(mx_specs))


def simd_reduce_mean(in1, dim=None, keepdim=False, mx_specs=None):
    mx_assert_test(mx_specs)
    if dim is None:
        dim = list(range(in1.ndim))
    if mx_specs is None:
        return torch_mean(in1, dim, keepdim=keepdim)
    mx_specs = apply_mx_specs(mx_specs)
    dim = dim if type(dim) is list else [dim]
    count = np.prod([in1.shape[i] for i in dim])
    return SIMDMul.apply(SIMDReduceSum.apply(in1, dim, keepdim, mx_specs), 1 / count, mx_specs)


def simd_norm(in1, keepdim=False, mx_specs=None):
    """Frobenius norm sqrt(sum(x^2)) (torch.linalg.norm without further arguments)."""
    mx_assert_test(mx_specs)
    if mx_specs is None:
        return torch.linalg.norm(in1, keepdim=keepdim)
    mx_specs = apply_mx_specs(mx_specs)
    sq = SIMDSquare.apply(in1, mx_specs)
    return SIMDSqrt.apply(SIMDReduceSum.apply(sq, list(range(sq.ndim)), keepdim, mx_specs), mx_specs)
