"""The separate-steps form of LayerNorm and RMSNorm over the last axis: what the layers run when the
fused row kernels do not cover a case (CPU tensors, fp16, long or odd rows), as chains of vector ops
with the elementwise quantizer after each.  Both forms hand the backward pass the same two tensors:
the normalized input z and one statistic per row (LayerNorm: var + eps; RMSNorm: 1 / rms).
The order of the steps is the reference's (mx/norm_utils.py:25-114, 188-258, mx/layernorm.py:100-168):
every step is rounded, so another order gives other bits."""
from .vector_ops import (vec_add, vec_div, vec_mul, vec_recip, vec_reduce_mean, vec_sqrt, vec_sub)


def layer_norm_rows(x, weight, bias, eps, specs):
    """x, weight, bias already quantized.  Returns (weight * z + bias, z, var + eps)."""
    shift = vec_sub(x, vec_reduce_mean(x, [-1], keepdim=True, mx_specs=specs), mx_specs=specs)
    var_eps = vec_add(vec_reduce_mean(vec_mul(shift, shift, mx_specs=specs), [-1], keepdim=True, mx_specs=specs),
                      eps, mx_specs=specs)
    z = vec_mul(shift, vec_recip(vec_sqrt(var_eps, mx_specs=specs), mx_specs=specs), mx_specs=specs)
    return vec_add(vec_mul(weight, z, mx_specs=specs), bias, mx_specs=specs), z, var_eps


def layer_norm_rows_grad_input(grad_output, weight, z, var_eps, specs):
    """grad_output already quantized.  With s = sqrt(var + eps) and u = g * w:
    d = u / s - z * mean(u * z * s) / (var + eps), then d - mean(d): the row mean is taken last."""
    u = vec_mul(grad_output, weight, mx_specs=specs)
    std = vec_sqrt(var_eps, mx_specs=specs)
    d = vec_mul(u, vec_div(1.0, std, mx_specs=specs), mx_specs=specs)
    t = vec_reduce_mean(vec_mul(vec_mul(u, z, mx_specs=specs), std, mx_specs=specs), [-1], keepdim=True, mx_specs=specs)
    t = vec_mul(t, vec_div(1.0, var_eps, mx_specs=specs), mx_specs=specs)
    d = vec_add(d, vec_mul(-t, z, mx_specs=specs), mx_specs=specs)
    return vec_add(d, -vec_reduce_mean(d, [-1], keepdim=True, mx_specs=specs), mx_specs=specs)


def rms_norm_rows(x, weight, bias, eps, specs):
    """x, weight, bias already quantized.  Returns (weight * z + bias, z = x / rms, 1 / rms)."""
    ms = vec_reduce_mean(vec_mul(x, x, mx_specs=specs), -1, keepdim=True, mx_specs=specs)
    rms_inv = vec_recip(vec_sqrt(vec_add(ms, eps, mx_specs=specs), mx_specs=specs), mx_specs=specs)
    z = vec_mul(x, rms_inv, mx_specs=specs)
    return vec_add(vec_mul(weight, z, mx_specs=specs), bias, mx_specs=specs), z, rms_inv


def rms_norm_rows_grad_input(grad_output, weight, z, rms_inv, specs):
    """grad_output already quantized: d = g * w / rms, result d - z * mean(d * z).  The last subtraction
    carries no mx_specs in the reference (mx/layernorm.py:166) and so is not quantized."""
    d = vec_mul(vec_mul(grad_output, weight, mx_specs=specs), rms_inv, mx_specs=specs)
    proj = vec_reduce_mean(vec_mul(d, z, mx_specs=specs), -1, keepdim=True, mx_specs=specs)
    return vec_sub(d, vec_mul(z, proj, mx_specs=specs))
