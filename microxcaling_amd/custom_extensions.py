"""The reference's native extension surface, served by the gfx950 library.

``funcs`` offers the seven callables of the reference's pybind module (mx/cpp/funcs.cpp:234-242)
with the same names, positional order, defaults and error type (RuntimeError).  GPU functions
take contiguous tensors on a HIP device and launch on torch's current stream for that device;
the two ``*_cpp`` functions take CPU tensors.  Outputs are new tensors; inputs are not modified.
"""
import math
import types

import torch

from . import _lib

_DTYPE = {torch.float32: _lib.DTYPE_F32, torch.float16: _lib.DTYPE_F16,
          torch.bfloat16: _lib.DTYPE_BF16}

# Extra flags passed to every native call; see set_exponent_mode.
_flags = 0


def set_exponent_mode(mode):
    """'torch' (default): exponents follow floor(log2(x)) as torch's CPU kernels evaluate it, so
    results are bit-identical to the reference's pure-PyTorch path (float32, bfloat16 and float16
    tensors; on 16-bit tensors every op is rounded to the tensor dtype, as that path does).
    'exact': bit-field exponents, which is what the reference's CUDA kernels compute; float16 tensors
    are widened to fp32 and rounded back once, as those kernels do (mx/cpp/mx.cuh:72,88)."""
    global _flags
    if mode == "torch":
        _flags = _flags & ~_lib.FLAG_EXACT_EXPONENT
    elif mode == "exact":
        _flags = _flags | _lib.FLAG_EXACT_EXPONENT
    else:
        raise ValueError("exponent mode must be 'torch' or 'exact'")


def set_general_form(on):
    """The softmax, norm and activation kernels skip the special cases of the bfloat16 quantizer for
    waves whose values all lie in a range where none can occur.  on=True switches that shortcut off
    (same results, slower): what the tests compare the shortcut with."""
    global _flags
    _flags = (_flags | _lib.FLAG_GENERAL_FORM) if on else (_flags & ~_lib.FLAG_GENERAL_FORM)


def _flags_value():
    return _flags


def _dtype_code(t, who):
    if t.dtype not in _DTYPE:
        raise RuntimeError("%s: Tensor dtype not supported (%s)" % (who, t.dtype))
    return _DTYPE[t.dtype]


def _check_gpu_input(t, name, who):
    """CHECK_INPUT of the reference (mx/cpp/funcs.h:9-11)."""
    if not t.is_cuda:
        raise RuntimeError("%s: %s must be a CUDA tensor" % (who, name))
    if not t.is_contiguous():
        raise RuntimeError("%s: %s must be contiguous" % (who, name))


def _collapse(shape, axis):
    pre = 1
    for n in shape[:axis]:
        pre *= n
    post = 1
    for n in shape[axis + 1:]:
        post *= n
    return pre, shape[axis], post


def _stream(t):
    return torch.cuda.current_stream(t.device).cuda_stream


def quantize_mx_by_tile_func_cuda(A, scale_bits, elem_ebits, elem_mbits, elem_max_norm, tile_size,
                                  axis, flush_fp32_subnorms=False, rmode=0):
    who = "quantize_mx_by_tile_func_cuda"
    _check_gpu_input(A, "A", who)
    if not (0 <= axis < A.dim()):
        raise RuntimeError("%s: axis exceeds input dimensions" % who)
    out = torch.empty_like(A)
    pre, n, post = _collapse(A.shape, axis)
    lib = _lib.gpu()
    with torch.cuda.device(A.device):
        rc = lib.mxq_quantize_mx_by_tile(A.data_ptr(), out.data_ptr(), _dtype_code(A, who), pre, n,
                                         post, scale_bits, elem_ebits, elem_mbits, elem_max_norm,
                                         tile_size, int(bool(flush_fp32_subnorms)), int(rmode),
                                         _flags, _stream(A))
    _lib.check(rc, lib)
    return out


def quantize_mx_func_cuda(A, scale_bits, elem_ebits, elem_mbits, elem_max_norm, max_values, axis,
                          flush_fp32_subnorms=False, rmode=0):
    who = "quantize_mx_func_cuda"
    _check_gpu_input(A, "A", who)
    if not (0 <= axis < A.dim()):
        raise RuntimeError("%s: axis exceeds input dimensions" % who)
    _check_gpu_input(max_values, "max_values", who)
    pre, n, post = _collapse(A.shape, axis)
    if max_values.dtype != A.dtype or max_values.numel() != pre * post:
        raise RuntimeError("%s: max_values must be the keepdim max of A over `axis`" % who)
    out = torch.empty_like(A)
    lib = _lib.gpu()
    with torch.cuda.device(A.device):
        rc = lib.mxq_quantize_mx_given_max(A.data_ptr(), out.data_ptr(), max_values.data_ptr(),
                                           _dtype_code(A, who), pre, n, post, scale_bits,
                                           elem_ebits, elem_mbits, elem_max_norm,
                                           int(bool(flush_fp32_subnorms)), int(rmode), _flags,
                                           _stream(A))
    _lib.check(rc, lib)
    return out


def quantize_elemwise_func_cuda(A, bits, exp_bits, max_norm, rmode=0, saturate_normals=False,
                                allow_denorm=True):
    who = "quantize_elemwise_func_cuda"
    _check_gpu_input(A, "A", who)
    out = torch.empty_like(A)
    lib = _lib.gpu()
    with torch.cuda.device(A.device):
        rc = lib.mxq_quantize_elemwise(A.data_ptr(), out.data_ptr(), _dtype_code(A, who),
                                       A.numel(), bits, exp_bits, max_norm, int(rmode),
                                       int(bool(saturate_normals)), int(bool(allow_denorm)),
                                       _flags, _stream(A))
    _lib.check(rc, lib)
    return out


def _reduce_inner(A, sym, who):
    _check_gpu_input(A, "A", who)
    if A.dtype != torch.float32:
        raise RuntimeError("%s: only float32 is supported" % who)
    if A.dim() < 1:
        raise RuntimeError("%s: needs at least one dimension" % who)
    inner = A.shape[-1]
    # the reference returns zeros(sizes[:-1]) carrying the input's requires_grad (mx/cpp/reduce.cu:24-28);
    # the kernel writes every element, so the fill launch is left out
    out = torch.empty(A.shape[:-1], dtype=A.dtype, device=A.device, requires_grad=A.requires_grad)
    rows = out.numel()
    lib = _lib.gpu()
    with torch.cuda.device(A.device):
        rc = getattr(lib, sym)(A.data_ptr(), out.data_ptr(), rows, inner, _stream(A))
    _lib.check(rc, lib)
    return out


def reduce_sum_inner_dim(A):
    return _reduce_inner(A, "mxq_reduce_sum_inner", "reduce_sum_inner_dim")


def reduce_max_inner_dim(A):
    return _reduce_inner(A, "mxq_reduce_max_inner", "reduce_max_inner_dim")


def _reduce_outer(A, sym, who):
    _check_gpu_input(A, "A", who)
    if A.dtype != torch.float32:
        raise RuntimeError("%s: only float32 is supported" % who)
    if A.dim() < 1:
        raise RuntimeError("%s: needs at least one dimension" % who)
    outer = A.shape[0]
    out = torch.empty(A.shape[1:], dtype=A.dtype, device=A.device)
    inner = out.numel()
    lib = _lib.gpu()
    ws_bytes = lib.mxq_reduce_outer_workspace_bytes(outer, inner)
    ws = torch.empty(max(ws_bytes, 16), dtype=torch.uint8, device=A.device)
    with torch.cuda.device(A.device):
        rc = getattr(lib, sym)(A.data_ptr(), out.data_ptr(), ws.data_ptr(), outer, inner,
                               _stream(A))
    _lib.check(rc, lib)
    return out


def reduce_sum_outer_dim(A):
    """Sum over axis 0 (not part of the reference's extension)."""
    return _reduce_outer(A, "mxq_reduce_sum_outer", "reduce_sum_outer_dim")


def reduce_max_outer_dim(A):
    """Max over axis 0, NaN-propagating (not part of the reference's extension)."""
    return _reduce_outer(A, "mxq_reduce_max_outer", "reduce_max_outer_dim")


# ---- CPU tensors -------------------------------------------------------------------------------
def _check_cpu_input(t, name, who):
    if t.is_cuda:
        raise RuntimeError("%s: %s must be a CPU tensor" % (who, name))
    if not t.is_contiguous():
        raise RuntimeError("%s: %s must be contiguous" % (who, name))


def quantize_mx_func_cpp(A, scale_bits, elem_ebits, elem_mbits, elem_max_norm, max_values, axis,
                         flush_fp32_subnorms, rmode=0):
    who = "quantize_mx_func_cpp"
    _check_cpu_input(A, "A", who)
    if not (1 <= A.dim() <= 5):
        raise RuntimeError("%s: number of dims outside of range [1,5]" % who)
    if not (0 <= axis < A.dim()):
        raise RuntimeError("%s: shared axis < 0 or shared axis >= ndim" % who)
    max_values = max_values.contiguous()
    pre, n, post = _collapse(A.shape, axis)
    if max_values.dtype != A.dtype or max_values.numel() != pre * post:
        raise RuntimeError("%s: max_values must be the keepdim max of A over `axis`" % who)
    out = torch.empty_like(A)
    lib = _lib.host()
    rc = lib.mxq_host_quantize_mx_given_max(A.data_ptr(), out.data_ptr(), max_values.data_ptr(),
                                            _dtype_code(A, who), pre, n, post, scale_bits,
                                            elem_ebits, elem_mbits, elem_max_norm,
                                            int(bool(flush_fp32_subnorms)), int(rmode), _flags)
    _lib.check(rc, lib, "mxq_host_last_error")
    return out


def quantize_elemwise_func_cpp(input, bits, exp_bits, max_norm, rmode=0, saturate_normals=False,
                               allow_denorm=True):
    who = "quantize_elemwise_func_cpp"
    _check_cpu_input(input, "input", who)
    out = torch.empty_like(input)
    lib = _lib.host()
    rc = lib.mxq_host_quantize_elemwise(input.data_ptr(), out.data_ptr(), _dtype_code(input, who),
                                        input.numel(), bits, exp_bits, max_norm, int(rmode),
                                        int(bool(saturate_normals)), int(bool(allow_denorm)),
                                        _flags)
    _lib.check(rc, lib, "mxq_host_last_error")
    return out


def quantize_mx_by_tile_func_cpp(A, scale_bits, elem_ebits, elem_mbits, elem_max_norm, tile_size,
                                 axis, flush_fp32_subnorms=False, rmode=0, round_every_op=False):
    """CPU twin of quantize_mx_by_tile_func_cuda (not in the reference): the kernels' arithmetic
    on the host."""
    who = "quantize_mx_by_tile_func_cpp"
    _check_cpu_input(A, "A", who)
    if not (0 <= axis < A.dim()):
        raise RuntimeError("%s: axis exceeds input dimensions" % who)
    pre, n, post = _collapse(A.shape, axis)
    out = torch.empty_like(A)
    lib = _lib.host()
    flags = _flags | (_lib.HOST_FLAG_ROUND_EVERY_OP if round_every_op else 0)
    rc = lib.mxq_host_quantize_mx_by_tile(A.data_ptr(), out.data_ptr(), _dtype_code(A, who), pre, n,
                                          post, scale_bits, elem_ebits, elem_mbits, elem_max_norm,
                                          tile_size, int(bool(flush_fp32_subnorms)), int(rmode),
                                          flags)
    _lib.check(rc, lib, "mxq_host_last_error")
    return out


def _axes_extents(shape, axes, who):
    """(outer_0, shared_0, outer_1, ..., shared_n-1, outer_n) for sorted, distinct axes, as a ctypes
    int64 array."""
    import ctypes
    axes = list(axes)
    if not 1 <= len(axes) <= 3 or sorted(set(axes)) != axes or not all(0 <= a < len(shape) for a in axes):
        raise RuntimeError("%s: axes must be one to three distinct, sorted, valid dimensions" % who)
    ext, lo = [], 0
    for a in axes:
        ext += [math.prod(shape[lo:a]), int(shape[a])]
        lo = a + 1
    ext.append(math.prod(shape[lo:]))
    return (ctypes.c_int64 * len(ext))(*ext)


def quantize_mx_axes_func_cuda(A, scale_bits, elem_ebits, elem_mbits, elem_max_norm, tile_size, axes,
                               flush_fp32_subnorms=False, rmode=0):
    """MX quantization with the exponent shared over the blocks of several axes at once (tiles of
    tile_size positions of every axis in `axes`; tile_size <= 0: whole axes).  Not in the
    reference's extension, which takes one axis (mx/mx_ops.py:240-246)."""
    who = "quantize_mx_axes_func_cuda"
    _check_gpu_input(A, "A", who)
    ext = _axes_extents(A.shape, axes, who)
    out = torch.empty_like(A)
    lib = _lib.gpu()
    with torch.cuda.device(A.device):
        rc = lib.mxq_quantize_mx_axes(A.data_ptr(), out.data_ptr(), _dtype_code(A, who), len(axes), ext,
                                      scale_bits, elem_ebits, elem_mbits, elem_max_norm, tile_size,
                                      int(bool(flush_fp32_subnorms)), int(rmode), _flags, _stream(A))
    _lib.check(rc, lib)
    return out


def quantize_mx_axes_func_cpp(A, scale_bits, elem_ebits, elem_mbits, elem_max_norm, tile_size, axes,
                              flush_fp32_subnorms=False, rmode=0):
    """CPU twin of quantize_mx_axes_func_cuda."""
    who = "quantize_mx_axes_func_cpp"
    _check_cpu_input(A, "A", who)
    ext = _axes_extents(A.shape, axes, who)
    out = torch.empty_like(A)
    lib = _lib.host()
    rc = lib.mxq_host_quantize_mx_axes(A.data_ptr(), out.data_ptr(), _dtype_code(A, who), len(axes), ext,
                                       scale_bits, elem_ebits, elem_mbits, elem_max_norm, tile_size,
                                       int(bool(flush_fp32_subnorms)), int(rmode), _flags)
    _lib.check(rc, lib, "mxq_host_last_error")
    return out


def _check_noise(A, noise, who):
    if noise.dtype != A.dtype or noise.shape != A.shape or noise.device != A.device or not noise.is_contiguous():
        raise RuntimeError("%s: noise must be a contiguous tensor like A (same shape, dtype, device)" % who)


def quantize_elemwise_dither_func(A, noise, bits, exp_bits, max_norm, saturate_normals=False,
                                  allow_denorm=True):
    """round='dither' (mx/elemwise_ops.py:57-59) for CPU or GPU tensors: floor(scaled value + noise),
    noise in [0, 1) like torch.rand_like(A).  Not in the reference's extension (pure path only)."""
    who = "quantize_elemwise_dither_func"
    out = torch.empty_like(A)
    args = (_dtype_code(A, who), A.numel(), bits, exp_bits, max_norm, int(bool(saturate_normals)),
            int(bool(allow_denorm)), _flags)
    if A.is_cuda:
        _check_gpu_input(A, "A", who)
        _check_noise(A, noise, who)
        lib = _lib.gpu()
        with torch.cuda.device(A.device):
            rc = lib.mxq_quantize_elemwise_dither(A.data_ptr(), noise.data_ptr(), out.data_ptr(), *args, _stream(A))
        _lib.check(rc, lib)
    else:
        _check_cpu_input(A, "A", who)
        _check_noise(A, noise, who)
        lib = _lib.host()
        rc = lib.mxq_host_quantize_elemwise_dither(A.data_ptr(), noise.data_ptr(), out.data_ptr(), *args)
        _lib.check(rc, lib, "mxq_host_last_error")
    return out


def quantize_mx_dither_by_tile_func(A, noise, scale_bits, elem_ebits, elem_mbits, elem_max_norm, tile_size,
                                    axis, flush_fp32_subnorms=False):
    """MX quantization with round='dither' for CPU or GPU tensors; see quantize_elemwise_dither_func."""
    who = "quantize_mx_dither_by_tile_func"
    if not (0 <= axis < A.dim()):
        raise RuntimeError("%s: axis exceeds input dimensions" % who)
    pre, n, post = _collapse(A.shape, axis)
    out = torch.empty_like(A)
    args = (_dtype_code(A, who), pre, n, post, scale_bits, elem_ebits, elem_mbits, elem_max_norm, tile_size,
            int(bool(flush_fp32_subnorms)), _flags)
    if A.is_cuda:
        _check_gpu_input(A, "A", who)
        _check_noise(A, noise, who)
        lib = _lib.gpu()
        with torch.cuda.device(A.device):
            rc = lib.mxq_quantize_mx_dither_by_tile(A.data_ptr(), noise.data_ptr(), out.data_ptr(), *args, _stream(A))
        _lib.check(rc, lib)
    else:
        _check_cpu_input(A, "A", who)
        _check_noise(A, noise, who)
        lib = _lib.host()
        rc = lib.mxq_host_quantize_mx_dither_by_tile(A.data_ptr(), noise.data_ptr(), out.data_ptr(), *args)
        _lib.check(rc, lib, "mxq_host_last_error")
    return out


funcs = types.SimpleNamespace(
    quantize_mx_func_cpp=quantize_mx_func_cpp,
    quantize_elemwise_func_cpp=quantize_elemwise_func_cpp,
    quantize_mx_func_cuda=quantize_mx_func_cuda,
    quantize_mx_by_tile_func_cuda=quantize_mx_by_tile_func_cuda,
    quantize_elemwise_func_cuda=quantize_elemwise_func_cuda,
    reduce_sum_inner_dim=reduce_sum_inner_dim,
    reduce_max_inner_dim=reduce_max_inner_dim,
    # additions
    quantize_mx_by_tile_func_cpp=quantize_mx_by_tile_func_cpp,
    reduce_sum_outer_dim=reduce_sum_outer_dim,
    reduce_max_outer_dim=reduce_max_outer_dim,
    quantize_mx_axes_func_cuda=quantize_mx_axes_func_cuda,
    quantize_mx_axes_func_cpp=quantize_mx_axes_func_cpp,
    quantize_elemwise_dither_func=quantize_elemwise_dither_func,
    quantize_mx_dither_by_tile_func=quantize_mx_dither_by_tile_func,
)
