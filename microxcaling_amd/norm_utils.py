"""Shared arithmetic of the normalization layers (mx/norm_utils.py): mean / variance / scale as a
chain of vector ops, each followed by the elementwise quantizer, over arbitrary reduction axes
with optional channel groups."""
from .vector_ops import (vec_add, vec_div, vec_mul, vec_quantize, vec_recip, vec_reduce_mean,
                         vec_sqrt, vec_sub)


def _as_axes(axes):
    if isinstance(axes, list):
        return axes
    assert isinstance(axes, int)
    return [axes]


def _get_group_shape(x, axis, groups):
    """(N, C, ...) -> (N, groups, C // groups, ...) for GroupNorm (mx/norm_utils.py:11-22)."""
    C = x.shape[axis]
    assert C % groups == 0
    orig = list(x.shape)
    grouped = orig[:axis] + [groups, C // groups] + orig[axis + 1:]
    return orig, grouped


def _broadcast_shape(ndim, axis, size):
    shape = [1] * ndim
    shape[axis] = size
    return shape


def _norm_forward(x, axes, weight, bias, eps, mx_specs, groups=None, weight_axis=None,
                  use_running_stats=False, running_mean=None, running_var=None):
    """z = (x - mean) / sqrt(var + eps); output = z * weight + bias (mx/norm_utils.py:25-114).
    weight and bias are already quantized.  Returns
    (output, x_shift, x_norm, x_std_inv, x_mean, x_var + eps)."""
    s = mx_specs
    axes = _as_axes(axes)
    w_shape = None if weight_axis is None else _broadcast_shape(x.ndim, weight_axis, x.shape[weight_axis])
    if groups:
        orig_shape, grouped_shape = _get_group_shape(x, axes[0], groups)
        x = x.view(grouped_shape)
        axes = [a + 1 for a in axes]
    stat_shape = list(x.shape)
    stat_shape[0] = 1
    for a in axes:
        stat_shape[a] = 1

    if use_running_stats:
        assert running_mean is not None and running_var is not None
        x_mean = vec_quantize(running_mean, mx_specs=s).view(stat_shape)
        x_shift = vec_sub(x, x_mean, mx_specs=s)
        x_var = vec_quantize(running_var, mx_specs=s).view(stat_shape)
    else:
        x_mean = vec_reduce_mean(x, axes, keepdim=True, mx_specs=s)
        x_shift = vec_sub(x, x_mean, mx_specs=s)
        x_var = vec_reduce_mean(vec_mul(x_shift, x_shift, mx_specs=s), axes, keepdim=True, mx_specs=s)

    x_vare = vec_add(x_var, eps, mx_specs=s)
    x_std_inv = vec_recip(vec_sqrt(x_vare, mx_specs=s), mx_specs=s)
    x_norm = vec_mul(x_shift, x_std_inv, mx_specs=s)
    if groups:
        x_norm = x_norm.view(orig_shape)
    if w_shape is not None:
        weight, bias = weight.view(w_shape), bias.view(w_shape)
    output = vec_add(vec_mul(weight, x_norm, mx_specs=s), bias, mx_specs=s)
    return output, x_shift, x_norm, x_std_inv, x_mean, x_vare


def _norm_backward(grad_output, axes, weight, x_shift, x_std_inv, mx_specs, groups=None,
                   weight_axis=None):
    """Gradient with respect to the input from the saved shifted input and 1 / std
    (mx/norm_utils.py:117-185): dx = g w / std - mean(g w / std) - x_shift mean(g w x_shift) / std^3."""
    s = mx_specs
    axes = _as_axes(axes)
    if weight_axis is not None:
        weight = weight.view(_broadcast_shape(grad_output.ndim, weight_axis, grad_output.shape[weight_axis]))
    if groups:
        orig_shape, grouped_shape = _get_group_shape(grad_output, axes[0], groups)
        axes = [a + 1 for a in axes]
    dx_norm = vec_mul(grad_output, weight, mx_specs=s)
    if groups:
        dx_norm = dx_norm.view(grouped_shape)
    dx_shift = vec_mul(dx_norm, x_std_inv, mx_specs=s)
    dx_mean = vec_reduce_mean(-dx_shift, axes, keepdim=True, mx_specs=s)
    dx_std = vec_reduce_mean(vec_mul(dx_norm, x_shift, mx_specs=s), axes, keepdim=True, mx_specs=s)
    dx_std = vec_mul(dx_std, vec_mul(x_std_inv, x_std_inv, mx_specs=s), mx_specs=s)
    dx_std = vec_mul(dx_std, x_std_inv, mx_specs=s)
    dx = vec_add(dx_shift, vec_mul(-dx_std, x_shift, mx_specs=s), mx_specs=s)
    dx = vec_add(dx, dx_mean, mx_specs=s)
    return dx.view(orig_shape) if groups else dx


def _norm_backward_LN(grad_output, axes, weight, x_norm, x_var, mx_specs, groups=None,
                      weight_axis=None):
    """The same gradient from the saved *normalized* input and var + eps, the way LayerNorm saves
    them (mx/norm_utils.py:188-258); the mean term is taken last, over the other two."""
    s = mx_specs
    axes = _as_axes(axes)
    if weight_axis is not None:
        weight = weight.view(_broadcast_shape(grad_output.ndim, weight_axis, grad_output.shape[weight_axis]))
    if groups:
        orig_shape, grouped_shape = _get_group_shape(grad_output, axes[0], groups)
        axes = [a + 1 for a in axes]
    dx_norm = vec_mul(grad_output, weight, mx_specs=s)
    if groups:
        dx_norm = dx_norm.view(grouped_shape)
    x_std = vec_sqrt(x_var, mx_specs=s)
    x_std_inv = vec_div(1.0, x_std, mx_specs=s)
    dx_shift = vec_mul(dx_norm, x_std_inv, mx_specs=s)
    t = vec_mul(vec_mul(dx_norm, x_norm, mx_specs=s), x_std, mx_specs=s)
    t = vec_reduce_mean(t, axes, keepdim=True, mx_specs=s)
    t = vec_mul(t, vec_div(1.0, x_var, mx_specs=s), mx_specs=s)
    dx = vec_add(dx_shift, vec_mul(-t, x_norm, mx_specs=s), mx_specs=s)
    dx_mean = vec_reduce_mean(dx, axes, keepdim=True, mx_specs=s)
    dx = vec_add(dx, -dx_mean, mx_specs=s)
    return dx.view(orig_shape) if groups else dx
