"""pytest plugin (python -m pytest -p hip_on_host_plugin ...): the GPU-marked tests of the quantizers run
against the HIP kernels' own source, compiled for the host.

MXQ_HIP_ON_HOST_LIB names a build of microxcaling_amd/csrc/mxq_capi.hip (kernels of mxq_kernels.h included)
behind tests/cpp/emu/hip/hip_runtime.h: every kernel launch runs its workgroups one after another, the 256
lanes of a workgroup as 256 threads that meet at __syncthreads and at the lane exchanges of a wave.  This
plugin maps every cuda device to the CPU (as tests/cpu_dry_run_plugin.py does) and makes the package's
entry points for GPU *and* CPU tensors call that library through the same ctypes signatures as
libmxq_gfx950.so (tensors report is_cuda, so the layers take their fused paths) -- so the arithmetic, the vector handling, the lane exchanges and the launch geometry that
the tests exercise are those of the .hip sources, not of the host library.  Used by
tests/test_kernels_on_host.py only."""
import contextlib
import ctypes
import os
import types

import cpu_dry_run_plugin  # noqa: F401  (cuda -> cpu)
import torch

from microxcaling_amd import _lib
from microxcaling_amd import custom_extensions as ce

_emu = ctypes.CDLL(os.environ["MXQ_HIP_ON_HOST_LIB"])
for _name, (_res, _args) in _lib.GPU_SYMBOLS.items():
    if hasattr(_emu, _name):
        getattr(_emu, _name).restype = _res
        getattr(_emu, _name).argtypes = _args
_lib.gpu = lambda: _emu


def _contiguous_only(t, name, who):
    if not t.is_contiguous():
        raise RuntimeError("%s: %s must be contiguous" % (who, name))


ce._check_gpu_input = _contiguous_only
ce._stream = lambda t: None
from microxcaling_amd import fused  # noqa: E402  (its own names for the two, imported from custom_extensions)
fused._check_gpu_input = _contiguous_only
fused._stream = lambda t: None
torch.cuda.device = lambda *a, **k: contextlib.nullcontext()
torch.cuda.current_stream = lambda *a, **k: types.SimpleNamespace(cuda_stream=None)
# the layers choose their fused paths (packed operands, the MFMA GEMM, the attention-score kernel) by
# tensor.is_cuda: every tensor says yes, and the entry points behind those paths are the host build's
torch.Tensor.is_cuda = property(lambda self: True)

# CPU tensors take the GPU entry points (their pointers are host pointers, which is what the host build reads)
ce.funcs.quantize_mx_by_tile_func_cpp = lambda A, *a, round_every_op=False, **k: ce.quantize_mx_by_tile_func_cuda(A, *a, **k)
ce.funcs.quantize_mx_axes_func_cpp = ce.quantize_mx_axes_func_cuda
ce.funcs.quantize_elemwise_func_cpp = ce.quantize_elemwise_func_cuda
ce.funcs.quantize_mx_func_cpp = ce.quantize_mx_func_cuda


def _dither_elemwise(A, noise, bits, exp_bits, max_norm, saturate_normals=False, allow_denorm=True):
    who = "quantize_elemwise_dither_func"
    ce._check_noise(A, noise, who)
    out = torch.empty_like(A)
    rc = _emu.mxq_quantize_elemwise_dither(A.data_ptr(), noise.data_ptr(), out.data_ptr(), ce._dtype_code(A, who),
                                           A.numel(), bits, exp_bits, max_norm, int(bool(saturate_normals)),
                                           int(bool(allow_denorm)), ce._flags_value(), None)
    _lib.check(rc, _emu)
    return out


def _dither_mx(A, noise, scale_bits, elem_ebits, elem_mbits, elem_max_norm, tile_size, axis, flush_fp32_subnorms=False):
    who = "quantize_mx_dither_by_tile_func"
    ce._check_noise(A, noise, who)
    pre, n, post = ce._collapse(A.shape, axis)
    out = torch.empty_like(A)
    rc = _emu.mxq_quantize_mx_dither_by_tile(A.data_ptr(), noise.data_ptr(), out.data_ptr(), ce._dtype_code(A, who), pre, n,
                                             post, scale_bits, elem_ebits, elem_mbits, elem_max_norm, tile_size,
                                             int(bool(flush_fp32_subnorms)), ce._flags_value(), None)
    _lib.check(rc, _emu)
    return out


ce.funcs.quantize_elemwise_dither_func = _dither_elemwise
ce.funcs.quantize_mx_dither_by_tile_func = _dither_mx
