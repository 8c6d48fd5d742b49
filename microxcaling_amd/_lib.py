"""ctypes bindings to the two native libraries (declarations: include/mxq.h).

There is deliberately no fallback: a missing library or a failed call raises."""
import ctypes
import os

PKG = os.path.dirname(os.path.abspath(__file__))
GPU_LIB_PATH = os.path.join(PKG, "libmxq_gfx950.so")
HOST_LIB_PATH = os.path.join(PKG, "libmxq_host.so")

DTYPE_F32, DTYPE_F16, DTYPE_BF16 = 0, 1, 2
FLAG_EXACT_EXPONENT = 1
FLAG_GENERAL_FORM = 16
HOST_FLAG_ROUND_EVERY_OP = 2

_c_int, _c_i64, _c_f32, _c_ptr = ctypes.c_int, ctypes.c_int64, ctypes.c_float, ctypes.c_void_p

# name -> (restype, argtypes); kept in one place so tests can check the exports against the header
GPU_SYMBOLS = {
    "mxq_last_error": (ctypes.c_char_p, []),
    "mxq_version": (_c_int, []),
    "mxq_build_digest": (ctypes.c_char_p, []),
    "mxq_quantize_mx_by_tile": (_c_int, [_c_ptr, _c_ptr, _c_int, _c_i64, _c_i64, _c_i64, _c_int,
                                         _c_int, _c_int, _c_f32, _c_i64, _c_int, _c_int, _c_int,
                                         _c_ptr]),
    "mxq_quantize_mx_axes": (_c_int, [_c_ptr, _c_ptr, _c_int, _c_int, _c_ptr, _c_int, _c_int, _c_int, _c_f32,
                                      _c_i64, _c_int, _c_int, _c_int, _c_ptr]),
    "mxq_quantize_mx_dither_by_tile": (_c_int, [_c_ptr, _c_ptr, _c_ptr, _c_int, _c_i64, _c_i64, _c_i64, _c_int,
                                                _c_int, _c_int, _c_f32, _c_i64, _c_int, _c_int, _c_ptr]),
    "mxq_quantize_elemwise_dither": (_c_int, [_c_ptr, _c_ptr, _c_ptr, _c_int, _c_i64, _c_int, _c_int, _c_f32,
                                              _c_int, _c_int, _c_int, _c_ptr]),
    "mxq_quantize_mx_given_max": (_c_int, [_c_ptr, _c_ptr, _c_ptr, _c_int, _c_i64, _c_i64, _c_i64,
                                           _c_int, _c_int, _c_int, _c_f32, _c_int, _c_int, _c_int,
                                           _c_ptr]),
    "mxq_quantize_elemwise": (_c_int, [_c_ptr, _c_ptr, _c_int, _c_i64, _c_int, _c_int, _c_f32,
                                       _c_int, _c_int, _c_int, _c_int, _c_ptr]),
    "mxq_softmax_lastdim": (_c_int, [_c_ptr, _c_ptr, _c_int, _c_i64, _c_i64, _c_int, _c_int, _c_f32,
                                     _c_int, _c_int, _c_int, _c_int, _c_int, _c_ptr]),
    "mxq_norm_lastdim": (_c_int, [_c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_int, _c_i64, _c_i64,
                                  _c_f32, _c_int, _c_int, _c_int, _c_f32, _c_int, _c_int, _c_int, _c_ptr]),
    "mxq_activation_forward": (_c_int, [_c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_int, _c_i64, _c_int, _c_int,
                                        _c_int, _c_f32, _c_int, _c_int, _c_int, _c_int, _c_ptr]),
    "mxq_activation_backward": (_c_int, [_c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_int, _c_i64, _c_int, _c_int,
                                         _c_int, _c_f32, _c_int, _c_int, _c_int, _c_ptr]),
    "mxq_softmax_backward_lastdim": (_c_int, [_c_ptr, _c_ptr, _c_ptr, _c_int, _c_i64, _c_i64, _c_int,
                                              _c_int, _c_f32, _c_int, _c_int, _c_int, _c_int, _c_ptr]),
    "mxq_norm_backward_lastdim": (_c_int, [_c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_int, _c_i64, _c_i64,
                                           _c_int, _c_int, _c_int, _c_f32, _c_int, _c_int, _c_int, _c_ptr]),
    "mxq_norm_param_grads_workspace_bytes": (_c_i64, [_c_int, _c_i64, _c_i64]),
    "mxq_norm_param_grads": (_c_int, [_c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_i64, _c_int, _c_i64, _c_i64,
                                      _c_int, _c_int, _c_f32, _c_int, _c_int, _c_int, _c_ptr]),
    "mxq_binary_elemwise": (_c_int, [_c_ptr, _c_ptr, _c_f32, _c_int, _c_ptr, _c_int, _c_i64, _c_int, _c_int,
                                     _c_int, _c_f32, _c_int, _c_int, _c_int, _c_ptr]),
    "mxq_pack_mx": (_c_int, [_c_ptr, _c_ptr, _c_ptr, _c_int, _c_i64, _c_i64, _c_int, _c_int, _c_int,
                             _c_f32, _c_int, _c_int, _c_int, _c_ptr]),
    "mxq_pack_mx_t": (_c_int, [_c_ptr, _c_ptr, _c_ptr, _c_int, _c_i64, _c_i64, _c_i64, _c_int, _c_int,
                               _c_int, _c_f32, _c_int, _c_int, _c_int, _c_ptr]),
    "mxq_unpack_mx": (_c_int, [_c_ptr, _c_ptr, _c_int, _c_ptr, _c_int, _c_i64, _c_i64, _c_ptr]),
    "mxq_gemm_mx_nt": (_c_int, [_c_ptr, _c_ptr, _c_int, _c_ptr, _c_ptr, _c_int, _c_ptr, _c_ptr, _c_int,
                                _c_i64, _c_i64, _c_i64, _c_i64, _c_int, _c_ptr, _c_i64, _c_ptr]),
    "mxq_gemm_workspace_bytes": (_c_i64, [_c_i64, _c_i64, _c_i64, _c_i64, _c_int]),
    "mxq_gemm_plan": (_c_int, [_c_i64, _c_i64, _c_i64, _c_i64, _c_int]),
    "mxq_bmm_softmax_mx_nt": (_c_int, [_c_ptr, _c_ptr, _c_int, _c_ptr, _c_ptr, _c_int, _c_ptr, _c_i64, _c_i64,
                                       _c_i64, _c_i64, _c_int, _c_int, _c_ptr]),
    "mxq_reduce_sum_inner": (_c_int, [_c_ptr, _c_ptr, _c_i64, _c_i64, _c_ptr]),
    "mxq_reduce_max_inner": (_c_int, [_c_ptr, _c_ptr, _c_i64, _c_i64, _c_ptr]),
    "mxq_reduce_outer_workspace_bytes": (_c_i64, [_c_i64, _c_i64]),
    "mxq_reduce_sum_outer": (_c_int, [_c_ptr, _c_ptr, _c_ptr, _c_i64, _c_i64, _c_ptr]),
    "mxq_reduce_max_outer": (_c_int, [_c_ptr, _c_ptr, _c_ptr, _c_i64, _c_i64, _c_ptr]),
    "mxq_reduce_outer_static": (_c_int, [_c_ptr, _c_ptr, _c_int, _c_i64, _c_i64, _c_ptr]),
}
HOST_SYMBOLS = {
    "mxq_host_last_error": (ctypes.c_char_p, []),
    "mxq_host_build_digest": (ctypes.c_char_p, []),
    "mxq_host_quantize_mx_given_max": (_c_int, [_c_ptr, _c_ptr, _c_ptr, _c_int, _c_i64, _c_i64,
                                                _c_i64, _c_int, _c_int, _c_int, _c_f32, _c_int,
                                                _c_int, _c_int]),
    "mxq_host_quantize_mx_by_tile": (_c_int, [_c_ptr, _c_ptr, _c_int, _c_i64, _c_i64, _c_i64,
                                              _c_int, _c_int, _c_int, _c_f32, _c_i64, _c_int,
                                              _c_int, _c_int]),
    "mxq_host_quantize_mx_axes": (_c_int, [_c_ptr, _c_ptr, _c_int, _c_int, _c_ptr, _c_int, _c_int, _c_int,
                                           _c_f32, _c_i64, _c_int, _c_int, _c_int]),
    "mxq_host_quantize_mx_dither_by_tile": (_c_int, [_c_ptr, _c_ptr, _c_ptr, _c_int, _c_i64, _c_i64, _c_i64,
                                                     _c_int, _c_int, _c_int, _c_f32, _c_i64, _c_int, _c_int]),
    "mxq_host_quantize_elemwise_dither": (_c_int, [_c_ptr, _c_ptr, _c_ptr, _c_int, _c_i64, _c_int, _c_int,
                                                   _c_f32, _c_int, _c_int, _c_int]),
    "mxq_host_quantize_elemwise": (_c_int, [_c_ptr, _c_ptr, _c_int, _c_i64, _c_int, _c_int, _c_f32,
                                            _c_int, _c_int, _c_int, _c_int]),
}

_gpu = None
_host = None


def _load(path, symbols, what):
    if not os.path.exists(path):
        raise RuntimeError(
            "%s not found at %s: build it with `python -m microxcaling_amd.build_ext` "
            "(there is no fallback implementation)" % (what, path))
    lib = ctypes.CDLL(path)
    for name, (res, args) in symbols.items():
        fn = getattr(lib, name)          # AttributeError if the export is missing
        fn.restype = res
        fn.argtypes = args
    return lib


def gpu():
    """libmxq_gfx950.so (HIP kernels)."""
    global _gpu
    if _gpu is None:
        _gpu = _load(GPU_LIB_PATH, GPU_SYMBOLS, "the gfx950 kernel library")
    return _gpu


def host():
    """libmxq_host.so (CPU tensors)."""
    global _host
    if _host is None:
        _host = _load(HOST_LIB_PATH, HOST_SYMBOLS, "the host quantization library")
    return _host


def check(rc, lib, err_fn="mxq_last_error"):
    if rc != 0:
        raise RuntimeError(getattr(lib, err_fn)().decode())
