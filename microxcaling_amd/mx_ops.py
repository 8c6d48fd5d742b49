"""MX block quantization: the call surface of the reference's mx/mx_ops.py, served by the native
kernels.

One shared 2^k scale per `block_size` consecutive elements along one axis; elements are rounded to
`elem_format` relative to that scale and returned in the input dtype ("fake quantization").

Differences from the reference, on purpose:
  * every case -- any axis, any block size, ragged last block, an exponent shared over the blocks
    of up to three axes at once -- is one kernel launch (the reference reshapes, pads and takes a
    separate max for block sizes above 32 on the last axis, and serves several axes on its
    pure-PyTorch path only, mx/mx_ops.py:226-263); results are bit-identical to its pure-PyTorch
    path either way, so ``custom_cuda`` is accepted but does not change the result;
  * ``round='dither'`` draws its noise with torch.rand_like like the reference and runs natively
    (single axis).
"""
import torch

from .specs import mx_assert_test
from .formats import ElemFormat, RoundingMode, _get_format_params
from .elemwise_ops import _native_round


def _dither_noise(A, axes, block_size):
    """One uniform [0, 1) number per element, the ones the reference's torch.rand_like hands the same
    elements under the same generator state.  The reference draws inside the element quantizer, i.e. for
    the tensor already padded to whole blocks (mx/mx_ops.py:226-229, 285-288, mx/elemwise_ops.py:58): when
    an axis is not a multiple of block_size the draw has the padded shape -- the padding's numbers are
    drawn and dropped, so that every real element meets the same number as there (on a GPU the number an
    element gets depends on the size of the draw, not only on its position)."""
    shape = list(A.shape)
    if block_size > 0:
        for ax in axes:
            shape[ax] = -(-shape[ax] // block_size) * block_size
    if shape == list(A.shape):
        return torch.rand_like(A, requires_grad=False)
    noise = torch.rand(shape, dtype=A.dtype, device=A.device)
    for ax in axes:
        noise = noise.narrow(ax, 0, A.shape[ax])
    return noise.contiguous()


def _quantize_mx(A, scale_bits, elem_format, shared_exp_method="max", axes=None, block_size=0,
                 round="nearest", flush_fp32_subnorms=False, custom_cuda=False):
    """Same contract as mx/mx_ops.py:173-298."""
    if elem_format is None:
        return A
    assert scale_bits > 0
    if axes is None:
        raise Exception("axes required in order to determine which dimension to apply "
                        "block size to")
    axes = [axes] if type(axes) == int else list(axes)
    axes = [x + A.ndim if x < 0 else x for x in axes]
    # the reference normalizes a negative axis a second time further down (mx/mx_ops.py:193-194, 105): axes=[-2]
    # on a 1-D tensor, which its linear layer's backward pass asks for (mx/linear.py:124-137), means axis 0
    axes = [x + A.ndim if -A.ndim <= x < 0 else x for x in axes]
    axes = sorted(axes)
    if len(axes) == 0 or len(set(axes)) != len(axes):
        raise ValueError("axes must name at least one dimension, each once")
    if len(axes) > 3:
        raise NotImplementedError("the native kernels share an exponent over at most three axes")
    rmode = None if round == "dither" else _native_round(round)
    ebits, mbits, _, max_norm, _ = _get_format_params(elem_format)

    if shared_exp_method == "none":          # an exponent per element = blocks of one
        tile = 1
    elif shared_exp_method == "max":
        tile = block_size if block_size > 0 else 0      # 0: the whole axis is one block
    else:
        raise Exception("Unrecognized shared exponent selection method %s" % shared_exp_method)

    from . import custom_extensions as ce
    A = A.contiguous()
    if round == "dither":
        # stochastic rounding: floor(scaled value + u), u from torch's generator like the reference's
        # torch.rand_like (mx/elemwise_ops.py:58)
        if len(axes) > 1 and tile != 1:
            raise NotImplementedError("round='dither' with an exponent shared over several axes")
        if A.device.type not in ("cuda", "cpu"):
            raise ValueError("Unrecognized device type %s" % A.device.type)
        return ce.funcs.quantize_mx_dither_by_tile_func(A, _dither_noise(A, axes, block_size), scale_bits,
                                                        ebits, mbits, max_norm, tile, axes[-1], flush_fp32_subnorms)
    if len(axes) > 1 and tile != 1:          # one exponent per tile of tile x tile (x tile) elements
        fn = {"cuda": ce.funcs.quantize_mx_axes_func_cuda, "cpu": ce.funcs.quantize_mx_axes_func_cpp}.get(A.device.type)
        if fn is None:
            raise ValueError("Unrecognized device type %s" % A.device.type)
        return fn(A, scale_bits, ebits, mbits, max_norm, tile, axes, flush_fp32_subnorms, rmode)
    axis = axes[-1]                          # blocks of one element: any axis serves
    if A.device.type == "cuda":
        return ce.funcs.quantize_mx_by_tile_func_cuda(
            A, scale_bits, ebits, mbits, max_norm, tile, axis, flush_fp32_subnorms, rmode)
    if A.device.type == "cpu":
        return ce.funcs.quantize_mx_by_tile_func_cpp(
            A, scale_bits, ebits, mbits, max_norm, tile, axis, flush_fp32_subnorms, rmode)
    raise ValueError("Unrecognized device type %s" % A.device.type)


def quantize_mx_op(A, mx_specs: dict, elem_format=None, block_size=None, axes=None,
                   round="nearest", expand_and_reshape=False):
    """Spec-driven entry point used by every MX layer (mx/mx_ops.py:301-331)."""
    mx_assert_test(mx_specs)
    if elem_format is None:
        return A
    if type(elem_format) is str:
        elem_format = ElemFormat.from_str(elem_format)
    if block_size is None:
        block_size = mx_specs["block_size"]
    scale_bits = mx_specs["scale_bits"] if mx_specs["scale_bits"] != 0 else 8
    return _quantize_mx(A, scale_bits, elem_format, block_size=block_size, axes=axes, round=round,
                        shared_exp_method=mx_specs["shared_exp_method"],
                        flush_fp32_subnorms=mx_specs["mx_flush_fp32_subnorms"],
                        custom_cuda=mx_specs["custom_cuda"])
