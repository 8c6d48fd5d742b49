"""CPU-side checks of the native code: both shared libraries load and export every symbol that
include/mxq.h declares; the kernels' scalar arithmetic (mxq_core.h, compiled for the host in
libmxq_host.so) is bit-identical to the oracle on exhaustive sweeps; the round-up-zone tables
agree with torch's CPU log2 on this machine.  No GPU compute happens here."""
import ctypes
import os
import subprocess
import re

import numpy as np
import pytest
import torch

from helpers import ROOT_DIR, assert_bits_equal, golden_inputs_module
from oracle import mx_oracle as O
from microxcaling_amd import _lib
from microxcaling_amd.custom_extensions import funcs
from microxcaling_amd.formats import _get_format_params
from microxcaling_amd.mx_ops import _quantize_mx
from microxcaling_amd.elemwise_ops import _quantize_elemwise_core

ROUNDS = ["nearest", "floor", "even"]
RMODE = {"nearest": 0, "floor": 1, "even": 2}
MX_FORMATS = ["fp8_e4m3", "fp8_e5m2", "fp6_e3m2", "fp6_e2m3", "fp4_e2m1", "int8", "int4", "int2"]


# ---- the C ABI ----------------------------------------------------------------------------------
def declared_symbols():
    text = open(os.path.join(ROOT_DIR, "include", "mxq.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(mxq_\w+)\s*\(", text)))


def test_header_declares_the_expected_entry_points():
    names = declared_symbols()
    for must in ("mxq_quantize_mx_by_tile", "mxq_quantize_mx_given_max", "mxq_quantize_elemwise",
                 "mxq_reduce_sum_inner", "mxq_reduce_max_inner", "mxq_last_error",
                 "mxq_host_quantize_mx_given_max", "mxq_host_quantize_elemwise"):
        assert must in names


def test_libraries_export_every_declared_symbol():
    assert os.path.exists(_lib.GPU_LIB_PATH), "run python -m microxcaling_amd.build_ext"
    gpu = ctypes.CDLL(_lib.GPU_LIB_PATH)          # loads without a GPU; nothing is launched
    host = ctypes.CDLL(_lib.HOST_LIB_PATH)
    for name in declared_symbols():
        lib = host if name.startswith("mxq_host_") else gpu
        assert hasattr(lib, name), "%s is declared in include/mxq.h but not exported" % name
    assert set(_lib.GPU_SYMBOLS) | set(_lib.HOST_SYMBOLS) == set(declared_symbols())


def test_every_translation_unit_compiles():
    """A front-end pass over every source of both libraries (seconds): a tree in which one file uses what
    another no longer defines does not get past this."""
    from microxcaling_amd import build_ext
    build_ext.check_sources()


def test_the_libraries_in_the_tree_are_built_from_the_sources_in_the_tree():
    """Both libraries carry the digest of the sources they were compiled from; it must be the digest of
    the source files next to them (otherwise: python -m microxcaling_amd.build_ext)."""
    from microxcaling_amd import build_ext
    want = build_ext.source_digest().encode()
    assert _lib.gpu().mxq_build_digest() == want, "libmxq_gfx950.so is stale: rebuild it"
    assert _lib.host().mxq_host_build_digest() == want, "libmxq_host.so is stale: rebuild it"


def test_kernels_of_the_built_library_fit_their_launch_shape():
    """From the code objects' own metadata: registers leave room for the waves each launch shape puts on
    a SIMD (512 per lane and SIMD, arch + accumulation), static LDS fits the 160 KB of a CU, and only the
    kernels named here keep anything in private (scratch) memory -- the streaming quantizers, packers,
    reductions and row kernels must not spill, since a spill in them is paid per element."""
    import re
    from microxcaling_amd import build_ext
    kernels = build_ext.kernel_resources()
    assert len(kernels) > 900

    def plain(k):                                        # _ZN12_GLOBAL__N_1<length><name>... -> name
        m = re.match(r"_ZN12_GLOBAL__N_1(\d+)", k["name"])
        return k["name"][m.end():m.end() + int(m.group(1))]

    names = {plain(k) for k in kernels}
    for want in ("mx_lastaxis_kernel", "mx_strided_kernel", "mx_strided_tile_kernel", "mx_axes_kernel", "elemwise_kernel",
                 "mx_pack_kernel", "mx_pack_t_kernel", "mx_unpack_kernel", "reduce_outer_kernel", "softmax_row_kernel",
                 "mx_gemm_nt_kernel", "mx_gemm_nt_kernel_256p", "mx_bmm_softmax_kernel"):
        assert want in names, want
    # name prefix -> bytes of private memory per lane that are known and accounted for: the large GEMM's fp32
    # epilogue keeps 8 loop-invariant address pairs there (written once per workgroup, read per tile after the
    # K loop), the scores kernel 6, one fp32 instantiation of the norm backward row kernel its row buffer
    allowed = {"mx_gemm_nt_kernel_256p": 68, "mx_bmm_softmax_kernel": 48, "norm_backward_row_kernel": 272}
    for k in kernels:
        name = plain(k)
        waves_per_simd = max(1, k["max_workgroup"] // 256)
        assert k["vgprs"] + k["agprs"] <= 512 // waves_per_simd, k
        assert k["lds"] <= 160 * 1024, k
        assert k["scratch"] <= allowed.get(name, 0), k
        if k["scratch"] == 0:
            assert k["vgpr_spills"] == 0, k


def test_gpu_entry_points_reject_bad_arguments_without_a_gpu():
    lib = _lib.gpu()
    assert lib.mxq_version() >= 100
    # argument errors are detected before anything touches the device
    rc = lib.mxq_quantize_mx_by_tile(None, None, 7, 1, 32, 1, 8, 4, 5, 448.0, 32, 0, 0, 0, None)
    assert rc == 1 and b"dtype" in lib.mxq_last_error()
    rc = lib.mxq_quantize_mx_by_tile(None, None, 0, 1, 32, 1, 9, 4, 5, 448.0, 32, 0, 0, 0, None)
    assert rc == 1 and b"scale_bits" in lib.mxq_last_error()
    rc = lib.mxq_quantize_elemwise(None, None, 0, 16, 30, 8, 1.0, 0, 0, 1, 0, None)
    assert rc == 1 and b"bits" in lib.mxq_last_error()
    rc = lib.mxq_quantize_elemwise(None, None, 0, 16, 9, 8, 1.0, 5, 0, 1, 0, None)
    assert rc == 1 and b"rounding" in lib.mxq_last_error()
    rc = lib.mxq_quantize_mx_by_tile(None, None, 0, 1, 32, 1, 8, 4, 5, 448.0, 32, 0, 0, 0, None)
    assert rc == 1 and b"null" in lib.mxq_last_error()
    assert lib.mxq_quantize_mx_by_tile(None, None, 0, 0, 32, 1, 8, 4, 5, 448.0, 32, 0, 0, 0, None) == 0
    assert lib.mxq_reduce_outer_workspace_bytes(16384, 8192) > 0
    # the entry points for several shared axes, dither, parameter gradients and the packing flags
    import ctypes
    ext = (ctypes.c_int64 * 5)(1, 64, 1, 64, 1)
    rc = lib.mxq_quantize_mx_axes(None, None, 0, 4, ext, 8, 4, 5, 448.0, 32, 0, 0, 0, None)
    assert rc == 1 and b"shared axes" in lib.mxq_last_error()
    rc = lib.mxq_quantize_mx_axes(None, None, 0, 2, ext, 8, 4, 5, 448.0, 32, 0, 0, 0, None)
    assert rc == 1 and b"null" in lib.mxq_last_error()
    ext0 = (ctypes.c_int64 * 5)(1, 64, 0, 64, 1)
    assert lib.mxq_quantize_mx_axes(None, None, 0, 2, ext0, 8, 4, 5, 448.0, 32, 0, 0, 0, None) == 0
    rc = lib.mxq_quantize_elemwise_dither(None, None, None, 0, 16, 9, 8, 1.0, 0, 1, 0, None)
    assert rc == 1 and b"null" in lib.mxq_last_error()
    rc = lib.mxq_quantize_mx_dither_by_tile(None, None, None, 0, 1, 32, 1, 9, 4, 5, 448.0, 32, 0, 0, None)
    assert rc == 1 and b"scale_bits" in lib.mxq_last_error()
    need = lib.mxq_norm_param_grads_workspace_bytes(2, 32768, 4096)
    assert need > 0 and need % (2 * 4096 * 4) == 0
    assert lib.mxq_norm_param_grads_workspace_bytes(2, 32768, 4100) == 0          # not a multiple of 16 bytes
    rc = lib.mxq_norm_param_grads(None, None, None, None, None, 0, 2, 8, 4100, 9, 8, 1.0, 0, 1, 0, None)
    assert rc == 1 and b"multiple" in lib.mxq_last_error()
    rc = lib.mxq_norm_param_grads(None, None, None, None, None, 0, 2, 8, 4096, 9, 8, 1.0, 0, 1, 0, None)
    assert rc == 1 and b"null" in lib.mxq_last_error()
    rc = lib.mxq_pack_mx(ctypes.c_void_p(16), ctypes.c_void_p(16), ctypes.c_void_p(16), 0, 4, 64, 8, 4, 5, 448.0,
                         0, 0, 32, None)                                         # pre-bfloat16 flag on an fp32 tensor
    assert rc == 1 and b"bf16" in lib.mxq_last_error()


def test_host_functions_reject_gpu_only_misuse():
    x = torch.zeros(4, 4)
    with pytest.raises(RuntimeError):
        funcs.quantize_mx_by_tile_func_cuda(x, 8, 4, 5, 448.0, 32, 1)        # CPU tensor
    with pytest.raises(RuntimeError):
        funcs.quantize_elemwise_func_cuda(x, 9, 8, 1.0)
    with pytest.raises(RuntimeError):
        funcs.reduce_sum_inner_dim(x)
    with pytest.raises(RuntimeError):
        funcs.quantize_mx_func_cpp(torch.zeros(2, 2, 2, 2, 2, 2), 8, 4, 5, 448.0,
                                   torch.zeros(1), 0, False)                  # ndim > 5
    with pytest.raises(NotImplementedError):
        _quantize_mx(x, 8, "fp8_e4m3", axes=[0, 1], block_size=2, round="dither")
    with pytest.raises(NotImplementedError):
        _quantize_mx(x, 8, "fp8_e4m3", axes=[-1], block_size=2, round="stochastic")
    with pytest.raises(NotImplementedError):
        _quantize_mx(torch.zeros(2, 2, 2, 2), 8, "fp8_e4m3", axes=[0, 1, 2, 3], block_size=2)
    with pytest.raises(ValueError):
        _quantize_mx(x, 8, "fp8_e4m3", axes=[1, -1], block_size=2)           # the same axis twice


# ---- round-up zones against torch's own log2 ----------------------------------------------------
def test_zone_tables_match_torch_log2_bf16():
    codes = torch.arange(1, 0x7F80, dtype=torch.int32).to(torch.int16).view(torch.bfloat16)
    want = torch.floor(torch.log2(codes)).float()
    # Read the kernels' floor(log2|x|) back through the quantizer: a block holding just x, int2
    # elements (values {0, +-1} x 2**E), floor rounding.
    y = _quantize_mx(codes.view(-1, 1), 8, "int2", axes=[1], block_size=1, round="floor").float()
    # int2 with shared exponent E: x / 2**E in [1, 2) floors to 1 when E is the true exponent, and
    # x / 2**(E+1) in [0.5, 1) floors to 0 when the zone pushed E up.
    true_k = torch.floor(torch.log2(codes.double())).float()
    got = torch.where(y.view(-1) == 0, true_k + 1, true_k)
    inrange = (want - 0).abs() <= 127                          # scale exponent clamps at +-127
    assert torch.equal(got[inrange], want[inrange])


def test_zone_tables_match_torch_log2_fp16():
    """Every positive finite fp16 code: the exponent the host library derives (bit field + zone table)
    is torch's floor(log2(x)) evaluated in fp16.  Read back as above; where the exponent comes out as
    16 the block scale 2**16 is Inf in fp16 and the block is NaN."""
    codes = torch.arange(1, 0x7C00, dtype=torch.int32).to(torch.int16).view(torch.float16)
    want = torch.floor(torch.log2(codes)).float()
    y = _quantize_mx(codes.view(-1, 1), 8, "int2", axes=[1], block_size=1, round="floor").float().view(-1)
    true_k = torch.floor(torch.log2(codes.double())).float()
    got = torch.where((y == 0) | y.isnan(), true_k + 1, true_k)
    assert (got != true_k).sum() > 50                           # the zones are there
    assert torch.equal(got, want)
    assert torch.equal(y.isnan(), want == 16)


def test_zone_tables_match_torch_log2_fp32():
    parts = []
    for be in range(1, 255):
        parts.append(((be << 23) + (1 << 23) - 1 - torch.arange(0, 128, dtype=torch.int64)))
    for k in range(-149, -126):                                  # subnormal binades, top codes
        hi = (1 << (k + 150)) - 1
        c = hi - torch.arange(0, 128, dtype=torch.int64)
        parts.append(c[c >= (1 << (k + 149))])
    x = torch.cat(parts).to(torch.int32).view(torch.float32)
    want = torch.floor(torch.log2(x))
    y = _quantize_mx(x.view(-1, 1), 8, "int2", axes=[1], block_size=1, round="floor")
    true_k = torch.floor(torch.log2(x.double())).float()
    got = torch.where(y.view(-1) == 0, true_k + 1, true_k)
    inrange = want.abs() <= 127
    assert inrange.sum() > 30000
    assert torch.equal(got[inrange], want[inrange])


# ---- exhaustive sweeps: host build of the kernel arithmetic vs the torch oracle ------------------
def all_bf16():
    return torch.arange(0, 65536, dtype=torch.int32).to(torch.int16).view(torch.bfloat16)


@pytest.mark.parametrize("bits,ebits,max_norm", [(9, 8, 2 ** 127 * 255 / 128), (12, 5, 65504.0),
                                                 (5, 4, 448.0), (4, 5, 57344.0), (3, 2, 6.0),
                                                 (8, 0, 127 / 64), (5, 8, 2 ** 127 * 15 / 8),
                                                 # more fraction bits than a bf16 tensor has
                                                 (10, 8, 2 ** 127 * 255 / 128), (16, 8, 3.0e38),
                                                 (9, 5, 65408.0), (10, 4, 480.0), (9, 0, 255 / 128)])
@pytest.mark.parametrize("rnd", ROUNDS)
def test_elementwise_every_bf16_code(bits, ebits, max_norm, rnd):
    x = all_bf16()
    for sat in (False, True):
        for den in (True, False):
            want = O.quantize_elemwise_core(x.clone(), bits, ebits, max_norm, round=rnd,
                                            saturate_normals=sat, allow_denorm=den)
            got = _quantize_elemwise_core(x.clone(), bits, ebits, max_norm, round=rnd,
                                          saturate_normals=sat, allow_denorm=den)
            assert_bits_equal(got, want, "sat=%s den=%s" % (sat, den))


def test_closed_form_bf16_to_bfloat16_nearest_every_code():
    """The closed form the fused softmax kernel uses for its commonest case (bf16 tensor, bfloat16,
    round-half-away) against the op-by-op oracle on all 65536 bf16 codes."""
    import ctypes
    from microxcaling_amd import _lib
    x = all_bf16().contiguous()
    out = torch.empty_like(x)
    lib = _lib.host()
    max_norm = 2 ** 127 * 255 / 128
    rc = lib.mxq_host_quantize_elemwise(x.data_ptr(), out.data_ptr(), 2, x.numel(), 9, 8, max_norm, 0, 0, 1, 4)
    assert rc == 0, lib.mxq_host_last_error()
    want = O.quantize_elemwise_core(x.clone(), 9, 8, max_norm, round="nearest",
                                    saturate_normals=False, allow_denorm=True)
    assert_bits_equal(out, want, "closed form")
    # the variant for exponentials, sums and quotients: +0 <= x < 2^127, +Inf, NaN
    codes = torch.cat([torch.arange(0, 0x7F00), torch.arange(0x7F80, 0x8000)]).to(torch.int16)
    xp = codes.view(torch.bfloat16).contiguous()
    outp = torch.empty_like(xp)
    rc = lib.mxq_host_quantize_elemwise(xp.data_ptr(), outp.data_ptr(), 2, xp.numel(), 9, 8, max_norm, 0, 0, 1, 4 | 8)
    assert rc == 0, lib.mxq_host_last_error()
    assert_bits_equal(outp, O.quantize_elemwise_core(xp.clone(), 9, 8, max_norm, round="nearest",
                                                     saturate_normals=False, allow_denorm=True), "nonneg")
    # and it refuses what it does not cover
    assert lib.mxq_host_quantize_elemwise(x.data_ptr(), out.data_ptr(), 2, x.numel(), 9, 8, max_norm, 2, 0, 1, 4) != 0
    assert lib.mxq_host_quantize_elemwise(x.data_ptr(), out.data_ptr(), 2, x.numel(), 9, 8, 1000.0, 0, 0, 1, 4) != 0


def fp32_probe_values():
    """Every (8 exponent, 9 mantissa)-bit value (the sweep of mx/tests/test_quantize_mx.py:52),
    the top 96 codes of every binade, specials and seeded random bit patterns."""
    e = torch.arange(0, 256, dtype=torch.int64).view(-1, 1)
    m = torch.arange(0, 512, dtype=torch.int64).view(1, -1)
    a = ((e << 23) | (m << 14)).reshape(-1)
    tops = ((torch.arange(0, 255, dtype=torch.int64).view(-1, 1) << 23) + (1 << 23) - 1
            - torch.arange(0, 96, dtype=torch.int64).view(1, -1)).reshape(-1)
    g = torch.Generator().manual_seed(5)
    r = torch.randint(0, 2 ** 31 - 1, (100000,), generator=g, dtype=torch.int64)
    c = torch.cat([a, tops[tops > 0], r])
    c = torch.cat([c, c | (1 << 31)])
    return c.to(torch.int32).view(torch.float32)


@pytest.mark.parametrize("bits,ebits,max_norm", [(9, 8, 2 ** 127 * 255 / 128), (12, 5, 65504.0),
                                                 (5, 4, 448.0), (8, 0, 127 / 64), (24, 8, 3.4028234663852886e38)])
@pytest.mark.parametrize("rnd", ROUNDS)
def test_elementwise_fp32_probes(bits, ebits, max_norm, rnd):
    x = fp32_probe_values()
    for sat, den in ((False, True), (True, False)):
        want = O.quantize_elemwise_core(x.clone(), bits, ebits, max_norm, round=rnd,
                                        saturate_normals=sat, allow_denorm=den)
        got = _quantize_elemwise_core(x.clone(), bits, ebits, max_norm, round=rnd,
                                      saturate_normals=sat, allow_denorm=den)
        assert_bits_equal(got, want, "sat=%s den=%s" % (sat, den))


def bf16_blocks(Mcode):
    """[n, 32] bf16 blocks: column 0 is the block maximum, the other 31 columns sweep every finite
    bf16 code whose magnitude does not exceed it."""
    codes = all_bf16()
    M = torch.tensor([Mcode], dtype=torch.int16).view(torch.bfloat16)
    sel = codes[torch.isfinite(codes.float()) & (codes.float().abs() <= M.float())]
    n = (sel.numel() + 30) // 31 * 31
    body = torch.cat([sel, torch.zeros(n - sel.numel(), dtype=torch.bfloat16)]).view(-1, 31)
    return torch.cat([M.expand(body.shape[0], 1), body], dim=1).contiguous()


# block maxima: powers of two and zone / top-of-binade mantissas across the whole exponent range
_MCODES = [(be << 7) | man for be in (0, 1, 2, 60, 110, 120, 124, 126, 127, 128, 130, 133, 140, 200,
                                      250, 254) for man in (0, 0x58, 0x7B, 0x7F)] + [1, 3, 0x40]


@pytest.mark.parametrize("fmt", MX_FORMATS)
@pytest.mark.parametrize("rnd", ROUNDS)
def test_mx_every_bf16_code_under_many_scales(fmt, rnd):
    ebits, mbits, _, max_norm, _ = _get_format_params(fmt)
    for Mcode in _MCODES:
        if Mcode == 0:
            continue
        x = bf16_blocks(Mcode)
        want = O.quantize_mx(x.clone(), 8, fmt, axes=[-1], block_size=32, round=rnd)
        got = _quantize_mx(x.clone(), 8, fmt, axes=[-1], block_size=32, round=rnd)
        assert_bits_equal(got, want, "max code 0x%04x" % Mcode)
        # the variant that rounds to bf16 after every op must agree with the lean one
        full = funcs.quantize_mx_by_tile_func_cpp(x.clone(), 8, ebits, mbits, max_norm, 32, 1, False,
                                                  RMODE[rnd], round_every_op=True)
        assert_bits_equal(full, want, "every-op variant, max code 0x%04x" % Mcode)


@pytest.mark.parametrize("fmt", ["fp8_e4m3", "fp4_e2m1", "int4"])
@pytest.mark.parametrize("rnd", ROUNDS)
@pytest.mark.parametrize("scale_bits,flush", [(8, False), (5, True), (5, False), (8, True)])
def test_mx_fp32_encoding_sweep(fmt, rnd, scale_bits, flush):
    """The reference's own sweep (mx/tests/test_quantize_mx.py:47-74): all 2^18 (8, 9)-bit values,
    block sizes 8 / 9 / 64."""
    e = torch.arange(0, 255, dtype=torch.int64).view(-1, 1)
    m = torch.arange(0, 512, dtype=torch.int64).view(1, -1)
    c = ((e << 23) | (m << 14)).reshape(-1)
    x = torch.cat([c, c | (1 << 31)]).to(torch.int32).view(torch.float32)
    for bs in (8, 9, 64):
        want = O.quantize_mx(x.clone(), scale_bits, fmt, axes=[-1], block_size=bs, round=rnd,
                             flush_fp32_subnorms=flush)
        got = _quantize_mx(x.clone(), scale_bits, fmt, axes=[-1], block_size=bs, round=rnd,
                           flush_fp32_subnorms=flush)
        assert_bits_equal(got, want, "block %d" % bs)


@pytest.mark.parametrize("fmt", MX_FORMATS)
@pytest.mark.parametrize("rnd", ROUNDS)
def test_mx_fp32_zone_blocks(fmt, rnd):
    gen = golden_inputs_module()
    x = gen.fp32_zone_cases()
    want = O.quantize_mx(x.clone(), 8, fmt, axes=[-1], block_size=32, round=rnd)
    got = _quantize_mx(x.clone(), 8, fmt, axes=[-1], block_size=32, round=rnd)
    assert_bits_equal(got, want)


def test_cpp_entry_points_follow_the_reference_call_pattern():
    """quantize_mx_func_cpp is called with the blocked view and its abs-max
    (mx/mx_ops.py:244-263)."""
    g = torch.Generator().manual_seed(9)
    x = torch.randn(6, 128, generator=g)
    ebits, mbits, _, max_norm, _ = _get_format_params("fp6_e3m2")
    xb = x.view(6, 4, 32)
    mv = xb.abs().max(dim=2, keepdim=True).values
    got = funcs.quantize_mx_func_cpp(xb.contiguous(), 8, ebits, mbits, max_norm, mv, 2, False, 0)
    want = O.quantize_mx(x, 8, "fp6_e3m2", axes=[-1], block_size=32)
    assert_bits_equal(got.view(6, 128), want)
    got = funcs.quantize_elemwise_func_cpp(x, 9, 8, 2 ** 127 * 255 / 128, 2, False, True)
    assert_bits_equal(got, x.to(torch.bfloat16).float())


@pytest.mark.parametrize("shape,axis,bs", [((3, 70, 5), 1, 32), ((4, 64), 0, 32), ((7, 90), 1, 9),
                                           ((6, 33), 1, 0), ((2, 40, 3, 4), 1, 32), ((65, 7), 0, 10)])
def test_mx_shapes_on_host(shape, axis, bs):
    g = torch.Generator().manual_seed(sum(shape))
    for dtype in (torch.float32, torch.bfloat16):
        x = (torch.randn(*shape, generator=g) * torch.exp(torch.randn(*shape, generator=g))).to(dtype)
        want = O.quantize_mx(x, 8, "fp8_e4m3", axes=[axis], block_size=bs)
        assert_bits_equal(_quantize_mx(x, 8, "fp8_e4m3", axes=[axis], block_size=bs), want)


MULTI_AXIS_CASES = [((70, 45), [-2, -1], 32), ((3, 40, 5, 33), [1, 3], 8), ((6, 10, 12), [0, 1, 2], 4),
                    ((5, 64, 64), [1, 2], 0), ((4, 7, 9), [2, 0], 32), ((2, 3, 4, 5, 6), [1, 2, 4], 2),
                    ((64, 96), [0, 1], 32)]


def tiles_as_rows(x, bs):
    """A 2-D tensor cut into bs x bs tiles (zero padded), one tile per row, and the way back."""
    R, C = x.shape
    Rp, Cp = -(-R // bs) * bs, -(-C // bs) * bs
    xp = torch.zeros(Rp, Cp, dtype=x.dtype)
    xp[:R, :C] = x
    rows = xp.reshape(Rp // bs, bs, Cp // bs, bs).permute(0, 2, 1, 3).reshape(-1, bs * bs)

    def back(y):
        return y.reshape(Rp // bs, Cp // bs, bs, bs).permute(0, 2, 1, 3).reshape(Rp, Cp)[:R, :C]
    return rows, back


@pytest.mark.parametrize("shape", [(64, 96), (70, 45), (31, 33)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_two_axis_blocks_are_single_axis_blocks_of_the_flattened_tile(shape, dtype):
    """An exponent shared over 32 x 32 tiles (mx/mx_ops.py:95-154 with two axes) is the single-axis
    quantization of each tile laid out as one row of 1024: pins the oracle's multi-axis blocking, and
    the host library's, to the single-axis path that the golden vectors cover."""
    g = torch.Generator().manual_seed(sum(shape))
    x = (torch.randn(*shape, generator=g) * torch.exp2(torch.randint(-15, 15, shape, generator=g).float())).to(dtype)
    rows, back = tiles_as_rows(x, 32)
    for fmt, rnd in (("fp8_e4m3", "nearest"), ("fp4_e2m1", "even"), ("int8", "floor")):
        want = back(O.quantize_mx(rows, 8, fmt, axes=[-1], block_size=1024, round=rnd))
        assert_bits_equal(O.quantize_mx(x, 8, fmt, axes=[0, 1], block_size=32, round=rnd), want, "oracle")
        assert_bits_equal(_quantize_mx(x, 8, fmt, axes=[0, 1], block_size=32, round=rnd), want, "host library")


@pytest.mark.parametrize("shape,axes,bs", MULTI_AXIS_CASES)
def test_mx_several_axes_on_host(shape, axes, bs):
    g = torch.Generator().manual_seed(sum(shape))
    for dtype in (torch.float32, torch.bfloat16):
        x = (torch.randn(*shape, generator=g) * torch.exp2(torch.randint(-12, 12, shape, generator=g).float())).to(dtype)
        x.view(-1)[3] = 0.0
        x.view(-1)[-1] = float("nan")
        for fmt, rnd in (("fp8_e4m3", "nearest"), ("fp6_e3m2", "floor"), ("fp4_e2m1", "even"), ("int8", "nearest")):
            want = O.quantize_mx(x, 8, fmt, axes=axes, block_size=bs, round=rnd)
            assert_bits_equal(_quantize_mx(x, 8, fmt, axes=axes, block_size=bs, round=rnd), want,
                              "%s %s %s" % (shape, fmt, rnd))
    # an exponent per element: the axes do not matter
    a = _quantize_mx(x, 8, "fp8_e4m3", shared_exp_method="none", axes=axes, block_size=bs)
    assert_bits_equal(a, O.quantize_mx(x, 8, "fp8_e4m3", axes=[-1], block_size=1))


def test_shared_exp_method_none_is_block_of_one():
    x = torch.randn(5, 16, generator=torch.Generator().manual_seed(2))
    a = _quantize_mx(x, 8, "fp8_e4m3", shared_exp_method="none", axes=[-1], block_size=4)
    b = O.quantize_mx(x, 8, "fp8_e4m3", axes=[-1], block_size=1)
    assert_bits_equal(a, b)


def test_direct_pack_codes_equal_the_encoded_rounded_values(tmp_path):
    """The pack kernels' shortcut (code from the rounded significand, no float value in between)
    against the long way, on the host, for all five code formats x fp32 / bf16 tensors x rounding
    modes: tests/cpp/pack_code_check.cpp exits non-zero on the first mismatch."""
    import shutil
    import subprocess
    cxx = shutil.which("g++") or shutil.which("c++")
    if cxx is None:
        pytest.skip("no host C++ compiler")
    exe = str(tmp_path / "pack_code_check")
    subprocess.run([cxx, "-O2", "-std=c++17", "-ffp-contract=off", "-I", os.path.join(ROOT_DIR, "include"),
                    "-I", os.path.join(ROOT_DIR, "microxcaling_amd", "csrc"), "-o", exe,
                    os.path.join(ROOT_DIR, "tests", "cpp", "pack_code_check.cpp")], check=True)
    out = subprocess.run([exe], check=True, capture_output=True, text=True, timeout=300).stdout
    assert out.count("inputs agree") == 30 and "MISMATCH" not in out
    # nearest and even are served by the shortcut (floor takes the round-up-zone variant)
    assert out.count("zone variant") == 10


@pytest.mark.parametrize("compiler", ["g++", "/opt/rocm/lib/llvm/bin/clang++"])
def test_fp16_conversions_of_the_scalar_core(tmp_path, compiler):
    """mxq_f16_bits / mxq_f16_value (the rounding after every op of an fp16 tensor) against torch's
    conversions: every fp16 code, both neighbours of every rounding boundary between two codes, the
    boundaries themselves, and a sweep of fp32 patterns.  g++ compiles the integer form, clang the
    _Float16 form."""
    import shutil
    import subprocess
    cxx = shutil.which(compiler)
    if cxx is None:
        pytest.skip("no " + compiler)
    codes = torch.arange(0, 65536, dtype=torch.int32).to(torch.int16).view(torch.float16)
    pos = codes[:0x7C00].float()
    mid = (pos[:-1].double() + pos[1:].double()) / 2                 # exact in fp32: one more bit
    mid = torch.cat([mid, torch.tensor([65520.0], dtype=torch.float64)]).float()
    mb = mid.view(torch.int32)
    sweep = torch.arange(0, 2 ** 32, 40961, dtype=torch.int64).to(torch.int32).view(torch.float32)
    x = torch.cat([codes.float(), mid, (mb - 1).view(torch.float32), (mb + 1).view(torch.float32), sweep])
    x = torch.cat([x, -x])
    src, hb, fb = (str(tmp_path / n) for n in ("x.bin", "h.bin", "f.bin"))
    x.numpy().tofile(src)
    exe = str(tmp_path / "f16_round_check")
    subprocess.run([cxx, "-O2", "-std=c++17", "-ffp-contract=off", "-I", os.path.join(ROOT_DIR, "include"),
                    "-I", os.path.join(ROOT_DIR, "microxcaling_amd", "csrc"), "-o", exe,
                    os.path.join(ROOT_DIR, "tests", "cpp", "f16_round_check.cpp")], check=True)
    subprocess.run([exe, src, hb, fb], check=True, capture_output=True, timeout=120)
    got_h = torch.from_numpy(np.fromfile(hb, dtype=np.int16)).view(torch.float16)
    got_f = torch.from_numpy(np.fromfile(fb, dtype=np.float32))
    assert_bits_equal(got_h, x.half(), "fp32 -> fp16")
    assert_bits_equal(got_f, x.half().float(), "fp16 -> fp32")


def test_host_quantizers_under_address_and_undefined_behaviour_sanitizers(tmp_path):
    """tests/cpp/host_abi_sanitize.cpp + mxq_host.cpp compiled with -fsanitize=address,undefined: eight
    seconds of random calls (empty and ragged shapes, tiles longer than the axis, several shared axes, all
    dtypes / formats / flags, now and then a call large enough for the library's threads to start) on buffers
    of exactly the described size; any read or write past an operand, signed overflow or misaligned access
    ends the run with a report.  (The same driver under -fsanitize=thread reports no race.)"""
    exe = str(tmp_path / "host_abi_sanitize")
    subprocess.run(["/opt/rocm/lib/llvm/bin/clang++", "-std=c++17", "-O1", "-gline-tables-only", "-fsanitize=address,undefined",
                    "-fno-sanitize-recover=undefined", "-ffp-contract=off", "-pthread", "-I" + os.path.join(ROOT_DIR, "include"),
                    "-I" + os.path.join(ROOT_DIR, "microxcaling_amd", "csrc"),
                    os.path.join(ROOT_DIR, "tests", "cpp", "host_abi_sanitize.cpp"),
                    os.path.join(ROOT_DIR, "microxcaling_amd", "csrc", "mxq_host.cpp"), "-o", exe],
                   check=True, capture_output=True, text=True, timeout=600)
    res = subprocess.run([exe, "8"], capture_output=True, text=True, timeout=300)
    assert res.returncode == 0 and res.stdout.startswith("ok "), (res.stdout[-2000:], res.stderr[-4000:])
    assert int(res.stdout.split()[1]) > 1000


def _build_gemm_addr_check(tmp_path, include_dir=None):
    import shutil
    import subprocess
    cxx = shutil.which("g++") or shutil.which("c++")
    if cxx is None:
        pytest.skip("no host C++ compiler")
    exe = str(tmp_path / "gemm_addr_check")
    subprocess.run([cxx, "-O2", "-std=c++17", "-I", os.path.join(ROOT_DIR, "include"),
                    "-I", include_dir or os.path.join(ROOT_DIR, "microxcaling_amd", "csrc"), "-o", exe,
                    os.path.join(ROOT_DIR, "tests", "cpp", "gemm_addr_check.cpp")], check=True)
    return exe


def test_gemm_copies_lds_image_schedule_and_stores_on_the_host(tmp_path):
    """tests/cpp/gemm_addr_check.cpp, through the address functions the kernels are compiled from
    (microxcaling_amd/csrc/mxq_gemm_addr.h): every 16- and 4-byte range of the tile copies of both GEMM
    kernels inside its operand (benchmark shapes, ragged M / N, K % 512 != 0, nibbles, batches, K
    splits); the 256 x 256 kernel's LDS replayed K step by K step (landing ranges, the bytes every
    fragment and scale read returns, copies against the barriers, registers against the MFMA groups);
    its output stores (every element once, by the lane that holds it, inside and aligned); the
    attention-score kernel's ring, waits, staging and stores.  Exits non-zero at the first violation."""
    import subprocess
    exe = _build_gemm_addr_check(tmp_path)
    res = subprocess.run([exe], capture_output=True, text=True, timeout=900)
    out = res.stdout
    assert res.returncode == 0, out[-2000:]
    for word in ("OUT OF BOUNDS", "LDS MODEL:", "STORES:", "SCORES:"):
        assert word not in out, out[-2000:]
    assert "byte ranges inside their operands" in out
    assert out.count("256 x 256 tiles") == 11 and out.count("128 x 128 tiles") == 20
    assert out.count("all as the MFMAs want them") == 11
    assert out.count("each once and in place") == 33 and out.count("scores kernel") == 6


def test_the_host_check_replays_the_kernels_the_library_would_launch(tmp_path):
    """tests/cpp/gemm_addr_check.cpp restates the launch rules (which shapes take the 256 x 256 kernel, how
    many K splits the others get) to know what to replay; the library answers the same questions without a
    GPU (mxq_gemm_plan, mxq_gemm_workspace_bytes).  For every shape of the check both must agree, or the
    replay would vouch for a kernel that is not the one launched."""
    exe = _build_gemm_addr_check(tmp_path)
    res = subprocess.run([exe, "--plans"], capture_output=True, text=True, timeout=60)
    assert res.returncode == 0
    lib = _lib.gpu()
    lib.mxq_gemm_plan.restype = ctypes.c_int
    lib.mxq_gemm_plan.argtypes = [ctypes.c_int64] * 4 + [ctypes.c_int]
    lib.mxq_gemm_workspace_bytes.restype = ctypes.c_int64
    lib.mxq_gemm_workspace_bytes.argtypes = [ctypes.c_int64] * 4 + [ctypes.c_int]
    E4M3, E2M1, LARGE, SPLIT, ONE_STEP, SMALL = 0, 4, 2, 1, 3, 0
    n = 0
    for line in res.stdout.splitlines():
        batch, M, N, K, nib, large, splits = (int(v) for v in line.split())
        kind = E2M1 if nib else E4M3
        plan = lib.mxq_gemm_plan(batch, M, N, K, kind)
        want = LARGE if large else SPLIT if splits > 1 else ONE_STEP if (K // 2 if nib else K) == 128 else SMALL
        assert plan == want, (line, plan)
        assert lib.mxq_gemm_workspace_bytes(batch, M, N, K, kind) == (0 if splits == 1 else splits * batch * M * N * 4), line
        n += 1
    assert n == 20


@pytest.mark.parametrize("what, old, new, says", [
    ("the step's barrier one group later",
     "constexpr int large_barrier_group(int ng) { return ng - 3; }",
     "constexpr int large_barrier_group(int ng) { return ng - 2; }", "LDS MODEL:"),
    ("copies behind the barrier aimed at the stage still being read",
     "return gi > large_barrier_group(ng) ? 2 : 1; }", "return 1; }", "LDS MODEL: copy issued into bytes that are read"),
    ("a copy instruction short per step",
     "return gi == 0 ? 2 : gi == 1 ? 1 : gi > large_barrier_group(ng) ? 3 : 0;",
     "return gi == 0 ? 2 : gi == 1 ? 1 : gi > large_barrier_group(ng) ? 2 : 0;", "LDS MODEL: a fragment read returns the wrong bytes"),
    ("code rows landing one row down",
     "(wave * 32 + (i & 3) * 8) * 128);", "(wave * 32 + (i & 3) * 8 + 1) * 128);", "LDS MODEL: copy lands outside its LDS region"),
    ("the exchanged pieces stored at the wrong columns",
     "return elems * (2 * ((lane >> 4) & 1) + (lane >> 5)); }", "return elems * (((lane >> 4) & 1) + 2 * (lane >> 5)); }",
     "STORES: a value is stored at another element's place"),
    ("another permutation of the B fragment rows",
     "(fi & 16) + ((fi & 4) << 1) + ((fi & 8) >> 1) + (fi & 3)", "(fi & 16) + (fi & 8) + (fi & 4) + (fi & 3)",
     "STORES: a lane's own columns are not where its registers belong"),
    ("score tiles dealt to the waves one by one",
     "return 8 * (i >> 1) + 2 * wave + (i & 1); }", "return 4 * i + wave; }", "SCORES:"),
    ("score copies fetching a neighbouring column",
     "(((lane & 7) ^ large_key(r)) * 16));\n}\n// where column col16 of tile row", "(((lane & 7) ^ large_key(r + 2)) * 16));\n}\n// where column col16 of tile row",
     "SCORES: a fragment read returns the wrong bytes"),
])
def test_the_host_check_notices_a_wrong_address_function(tmp_path, what, old, new, says):
    """The check above must be able to fail: the same program compiled against a copy of the address
    header with one function changed stops at the violation that change causes."""
    import subprocess
    src = open(os.path.join(ROOT_DIR, "microxcaling_amd", "csrc", "mxq_gemm_addr.h")).read()
    old, new = old.replace("\\n", "\n"), new.replace("\\n", "\n")
    assert src.count(old) == 1, what
    inc = tmp_path / "inc"
    inc.mkdir()
    (inc / "mxq_gemm_addr.h").write_text(src.replace(old, new))
    exe = _build_gemm_addr_check(tmp_path, str(inc))
    res = subprocess.run([exe], capture_output=True, text=True, timeout=900)
    assert res.returncode == 1 and says in res.stdout, (what, res.stdout[-1500:])


def test_dither_reproduces_the_reference_under_the_same_seed():
    """round='dither' on CPU tensors: the package draws its noise like the reference
    (torch.rand_like under torch's generator) and the host library rounds floor(s + noise): the
    reference's seeded outputs (tests/golden/reference_dither_vectors.npz) come out bit for bit."""
    from helpers import dither_cases
    from microxcaling_amd.elemwise_ops import _quantize_elemwise_core
    for kind, name, dtype, case_no, seed, case, x, want in dither_cases():
        torch.manual_seed(seed)
        if kind == "mx":
            fmt, axis, bs = case
            got = _quantize_mx(x.clone(), 8, fmt, axes=[axis], block_size=bs, round="dither")
        else:
            bits, eb, mn, sat = case
            got = _quantize_elemwise_core(x.clone(), bits, eb, mn, round="dither", saturate_normals=sat)
        assert_bits_equal(got, want, "%s %s %d" % (kind, name, case_no))


def test_dither_is_floor_or_ceiling_and_unbiased():
    x = torch.linspace(-3.9, 3.9, 4001)
    from microxcaling_amd.elemwise_ops import _quantize_elemwise_core
    torch.manual_seed(0)
    draws = torch.stack([_quantize_elemwise_core(x, 5, 4, 448.0, round="dither") for _ in range(400)])
    lo = _quantize_elemwise_core(x, 5, 4, 448.0, round="floor")              # toward zero
    step = torch.exp2(torch.floor(torch.log2(x.abs().clamp_min(2.0 ** -6))) - 3)
    hi = lo + torch.sign(x) * step
    assert ((draws == lo) | (draws == hi)).all()
    assert ((draws.mean(0) - x).abs() <= 0.2 * step).all()
