"""Batch normalization over (N, C, ...) inputs: same interface as the reference's mx/batchnorm.py."""
import torch
import torch.nn.functional as F

from .norm_utils import _norm_backward, _norm_forward
from .specs import apply_mx_specs, get_backwards_mx_specs, mx_assert_test
from .vector_ops import vec_add, vec_mul, vec_quantize, vec_reduce_sum

f_batch_norm = F.batch_norm


def _batch_axes(t):
    return [0] + list(range(2, t.ndim))


def _blend(running, new, momentum, specs):
    """(1 - momentum) * running + momentum * new, three quantized steps (mx/batchnorm.py:75-90)."""
    return vec_add(vec_mul(1 - momentum, running, mx_specs=specs),
                   vec_mul(momentum, new, mx_specs=specs), mx_specs=specs)


class BatchNormFunction(torch.autograd.Function):
    """y = (x - mean) / sqrt(var + eps) * gamma + beta per channel (axis 1).  Training: batch
    statistics, running statistics updated in place; evaluation: running statistics
    (mx/batchnorm.py:16-123)."""

    @staticmethod
    def forward(ctx, x, running_mean, running_var, weight, bias, is_training=False, momentum=0.1,
                eps=1e-5, mx_specs=None):
        if not is_training:
            assert running_mean is not None and running_var is not None
        s = mx_specs
        x = vec_quantize(x, mx_specs=s)
        bf_weight = vec_quantize(weight, mx_specs=s)
        bf_bias = vec_quantize(bias, mx_specs=s)
        C = x.shape[1]
        output, x_shift, x_norm, x_std_inv, x_mean, x_var = _norm_forward(
            x, _batch_axes(x), bf_weight, bf_bias, eps, s, weight_axis=1,
            use_running_stats=not is_training, running_mean=running_mean, running_var=running_var)
        if is_training and running_mean is not None:
            running_mean.copy_(_blend(running_mean, x_mean.view(C), momentum, s))
        if is_training and running_var is not None:
            running_var.copy_(_blend(running_var, x_var.view(C), momentum, s))
        ctx.save_for_backward(x_shift, x_norm, x_std_inv, bf_weight if s['quantize_backprop'] else weight)
        ctx.mx_specs = get_backwards_mx_specs(s)
        return output

    @staticmethod
    def backward(ctx, grad_output):
        x_shift, x_norm, x_std_inv, weight = ctx.saved_tensors
        s = ctx.mx_specs
        axes = _batch_axes(grad_output)
        g = vec_quantize(grad_output, mx_specs=s)
        grad_bias = vec_reduce_sum(g, axes, mx_specs=s)
        grad_weight = vec_reduce_sum(vec_mul(g, x_norm, mx_specs=s), axes, mx_specs=s)
        grad_input = _norm_backward(g, axes, weight, x_shift, x_std_inv, s, weight_axis=1)
        return (grad_input, None, None, grad_weight, grad_bias, None, None, None, None)


def batch_norm(x, running_mean, running_var, weight, bias, is_training=False, momentum=0.1,
               eps=1e-5, mx_specs=None):
    mx_assert_test(mx_specs)
    if mx_specs is None:
        return f_batch_norm(x, running_mean, running_var, weight, bias, is_training, momentum, eps)
    return BatchNormFunction.apply(x, running_mean, running_var, weight, bias, is_training, momentum,
                                   eps, apply_mx_specs(mx_specs))


class _BatchNorm(torch.nn.modules.batchnorm._BatchNorm):
    """torch's module bookkeeping (momentum, batch counter, which statistics to use) around
    batch_norm above (mx/batchnorm.py:142-219)."""

    def __init__(self, num_features, mx_specs=None, name=None, **kwargs):
        super().__init__(num_features, **kwargs)
        mx_assert_test(mx_specs)
        self.mx_none = mx_specs is None
        self.mx_specs = apply_mx_specs(mx_specs)
        self.name = name

    def forward(self, input):
        if self.mx_none:
            return super().forward(input)
        self._check_input_dim(input)
        factor = 0.0 if self.momentum is None else self.momentum
        if self.training and self.track_running_stats and self.num_batches_tracked is not None:
            self.num_batches_tracked += 1
            factor = 1.0 / float(self.num_batches_tracked) if self.momentum is None else self.momentum
        use_batch_stats = self.training or (self.running_mean is None and self.running_var is None)
        keep_running = not self.training or self.track_running_stats
        return batch_norm(input, self.running_mean if keep_running else None,
                          self.running_var if keep_running else None, self.weight, self.bias,
                          is_training=use_batch_stats, momentum=factor, eps=self.eps,
                          mx_specs=self.mx_specs)


def _checked(name, dims):
    def _check_input_dim(self, input):
        if input.dim() not in dims:
            raise ValueError('expected %s input (got %dD input)'
                             % (" or ".join("%dD" % d for d in dims), input.dim()))
    return type(name, (_BatchNorm,), {"_check_input_dim": _check_input_dim})


BatchNorm1d = _checked("BatchNorm1d", (2, 3))
BatchNorm2d = _checked("BatchNorm2d", (4,))
BatchNorm3d = _checked("BatchNorm3d", (5,))
