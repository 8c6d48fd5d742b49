"""Fused MX GEMM: operands are quantized straight into packed element codes + E8M0 block scales
and multiplied by the gfx950 scaled-MFMA kernel (include/mxq.h: mxq_pack_mx, mxq_gemm_mx_nt).

Compared with fake-quantizing and calling a dense GEMM (the reference's way, mx/linear.py:62-86)
the products are the same numbers -- code x code x 2^(scale_a + scale_b) -- accumulated in fp32 in
a different order, so results agree to accumulation tolerance, not bit for bit.
"""
import torch

from . import _lib
from .custom_extensions import _DTYPE, _check_gpu_input, _flags_value, _stream

# tensor dtypes whose layers take the fused path (fp16 tensors have no packed form in the default
# exponent mode, where every op is rounded to fp16, and stay on the separate steps)
_FUSED_DTYPES = (torch.float32, torch.bfloat16)
from .formats import ElemFormat, RoundingMode, _get_format_params

_PACKABLE = (ElemFormat.fp8_e4m3, ElemFormat.fp8_e5m2, ElemFormat.fp6_e3m2, ElemFormat.fp6_e2m3,
             ElemFormat.fp4)
GEMM_K_MULTIPLE = 128
# kinds of element codes (include/mxq.h MXQ_CODES_*): e4m3 bytes, e5m2 bytes, e2m1 nibbles
CODES_E4M3, CODES_E5M2, CODES_E2M3, CODES_E3M2, CODES_E2M1 = 0, 1, 2, 3, 4
_FLAG_PACK_NIBBLES, _FLAG_PACK_SIXBIT = 4, 8


def _as_format(fmt):
    if fmt is None:
        return None
    return ElemFormat.from_str(fmt) if type(fmt) is str else fmt


def _code_kind(fmt, nibbles, who):
    """`nibbles` = pack below 8 bits per element: fp4 as nibbles, fp6 as 6-bit codes."""
    if nibbles:
        if fmt == ElemFormat.fp4:
            return CODES_E2M1
        if fmt in (ElemFormat.fp6_e2m3, ElemFormat.fp6_e3m2):
            return CODES_E2M3 if fmt == ElemFormat.fp6_e2m3 else CODES_E3M2
        raise RuntimeError("%s: only fp4 elements pack into nibbles and fp6 elements into 6-bit "
                           "codes (got %s)" % (who, fmt))
    return CODES_E5M2 if fmt == ElemFormat.fp8_e5m2 else CODES_E4M3


def _code_bytes(K, kind):
    """Bytes of codes for K elements of a row."""
    kind = int(kind)
    return K // 2 if kind == CODES_E2M1 else K * 3 // 4 if kind in (CODES_E2M3, CODES_E3M2) else K


def _pack_flag(kind):
    return _FLAG_PACK_NIBBLES if kind == CODES_E2M1 else \
        _FLAG_PACK_SIXBIT if kind in (CODES_E2M3, CODES_E3M2) else 0


_FLAG_PRE_BFLOAT16 = 32


def pack_mx(A, elem_format, scale_bits=8, round="nearest", flush_fp32_subnorms=False, nibbles=False,
            pre_bfloat16=False):
    """MX-quantize A along its last axis (block 32) into (codes, scales, code_kind): codes uint8 of
    A's shape (one e4m3 / e5m2 byte per element) or, with nibbles=True, of half the last axis for
    fp4 (two e2m1 codes per byte, the lower index in the low nibble) and of 3/4 of it for fp6 (6-bit
    codes as a little-endian bit stream); scales uint8 with the last axis divided by 32.
    pre_bfloat16 (bf16 tensors): the elements first go through the elementwise bfloat16 quantizer
    with round-half-away, in the same pass."""
    who = "pack_mx"
    fmt = _as_format(elem_format)
    if fmt not in _PACKABLE:
        raise RuntimeError("%s: element format %s has no packed form" % (who, fmt))
    kind = _code_kind(fmt, nibbles, who)
    _check_gpu_input(A, "A", who)
    if A.dtype not in _DTYPE:
        raise RuntimeError("%s: Tensor dtype not supported (%s)" % (who, A.dtype))
    K = A.shape[-1]
    if A.dim() < 1 or K % 32 != 0:
        raise RuntimeError("%s: the last axis must be a multiple of 32" % who)
    ebits, mbits, _, max_norm, _ = _get_format_params(fmt)
    rows = A.numel() // K if K else 0
    codes = torch.empty(A.shape[:-1] + (_code_bytes(K, kind),), dtype=torch.uint8, device=A.device)
    scales = torch.empty(A.shape[:-1] + (K // 32,), dtype=torch.uint8, device=A.device)
    lib = _lib.gpu()
    with torch.cuda.device(A.device):
        rc = lib.mxq_pack_mx(A.data_ptr(), codes.data_ptr(), scales.data_ptr(), _DTYPE[A.dtype],
                             rows, K, scale_bits, ebits, mbits, max_norm,
                             int(bool(flush_fp32_subnorms)), int(RoundingMode[round]),
                             _flags_value() | _pack_flag(kind) | (_FLAG_PRE_BFLOAT16 if pre_bfloat16 else 0),
                             _stream(A))
    _lib.check(rc, lib)
    return codes, scales, kind


def pack_mx_t(A, elem_format, scale_bits=8, round="nearest", flush_fp32_subnorms=False, nibbles=False):
    """MX-quantize A (..., R, C) along its second-to-last axis (block 32) and transpose while
    packing: codes uint8 (..., C, R) (or (..., C, R / 2) e2m1 nibbles), scales uint8
    (..., C, R / 32) -- K-major for a contraction over R.  Returns (codes, scales, code_kind)."""
    who = "pack_mx_t"
    fmt = _as_format(elem_format)
    if fmt not in _PACKABLE:
        raise RuntimeError("%s: element format %s has no packed form" % (who, fmt))
    kind = _code_kind(fmt, nibbles, who)
    _check_gpu_input(A, "A", who)
    if A.dtype not in _DTYPE:
        raise RuntimeError("%s: Tensor dtype not supported (%s)" % (who, A.dtype))
    if A.dim() < 2:
        raise RuntimeError("%s: needs at least two axes" % who)
    R, C = A.shape[-2], A.shape[-1]
    if R % 32 != 0 or C % (8 // A.element_size()) != 0:
        raise RuntimeError("%s: shape %s: the second-to-last axis must be a multiple of 32 and the "
                           "last one of 8 bytes" % (who, tuple(A.shape)))
    ebits, mbits, _, max_norm, _ = _get_format_params(fmt)
    batch = A.numel() // (R * C) if R * C else 0
    codes = torch.empty(A.shape[:-2] + (C, _code_bytes(R, kind)), dtype=torch.uint8, device=A.device)
    scales = torch.empty(A.shape[:-2] + (C, R // 32), dtype=torch.uint8, device=A.device)
    lib = _lib.gpu()
    with torch.cuda.device(A.device):
        rc = lib.mxq_pack_mx_t(A.data_ptr(), codes.data_ptr(), scales.data_ptr(), _DTYPE[A.dtype],
                               batch, R, C, scale_bits, ebits, mbits, max_norm,
                               int(bool(flush_fp32_subnorms)), int(RoundingMode[round]),
                               _flags_value() | _pack_flag(kind), _stream(A))
    _lib.check(rc, lib)
    return codes, scales, kind


def _packed_k(codes, scales, kind, who):
    """Length of the quantized axis of a packed tensor, after checking that codes and scales fit."""
    K = scales.shape[-1] * 32
    if codes.shape[:-1] != scales.shape[:-1] or codes.shape[-1] != _code_bytes(K, kind):
        raise RuntimeError("%s: codes %s and scales %s do not belong together (code kind %d)"
                           % (who, tuple(codes.shape), tuple(scales.shape), int(kind)))
    return K


def unpack_mx(codes, scales, code_kind, dtype=torch.float32):
    """codes * 2^(scales - 127) as a tensor of `dtype` (255 in scales -> NaN block)."""
    who = "unpack_mx"
    _check_gpu_input(codes, "codes", who)
    _check_gpu_input(scales, "scales", who)
    K = _packed_k(codes, scales, code_kind, who)
    out = torch.empty(codes.shape[:-1] + (K,), dtype=dtype, device=codes.device)
    lib = _lib.gpu()
    with torch.cuda.device(codes.device):
        rc = lib.mxq_unpack_mx(codes.data_ptr(), scales.data_ptr(), int(code_kind),
                               out.data_ptr(), _DTYPE[dtype], out.numel() // K if K else 0, K,
                               _stream(codes))
    _lib.check(rc, lib)
    return out


def gemm_nt(a_packed, b_packed, out_dtype=torch.float32, bias=None, epilogue_quant=False):
    """C[b] = A[b] x B[b]^T (+ bias).  a_packed / b_packed = (codes, scales, code_kind) as returned
    by pack_mx, of a (batch, M, K) / (batch, N, K) or (M, K) / (N, K) tensor; e2m1 nibble codes need
    both operands in that form; bias: (N,) of out_dtype, added after the
    product has been rounded to out_dtype, the sum being rounded again.  epilogue_quant (bf16
    output only): also apply the bfloat16 / round-half-away elementwise quantization after the
    product and after the bias add."""
    who = "gemm_nt"
    (ac, asc, ae), (bc, bsc, be) = a_packed, b_packed
    for t, n in ((ac, "a codes"), (asc, "a scales"), (bc, "b codes"), (bsc, "b scales")):
        _check_gpu_input(t, n, who)
    K = _packed_k(ac, asc, ae, who)
    if ac.dim() != bc.dim() or ac.dim() not in (2, 3) or _packed_k(bc, bsc, be, who) != K \
            or ac.shape[:-2] != bc.shape[:-2]:
        raise RuntimeError("%s: operand shapes %s and %s do not match" % (who, tuple(ac.shape),
                                                                          tuple(bc.shape)))
    batch = ac.shape[0] if ac.dim() == 3 else 1
    M, N = ac.shape[-2], bc.shape[-2]
    if bias is not None:
        _check_gpu_input(bias, "bias", who)
        if bias.dtype != out_dtype or bias.numel() != N:
            raise RuntimeError("%s: bias must hold N values of the output dtype" % who)
    out = torch.empty(ac.shape[:-2] + (M, N), dtype=out_dtype, device=ac.device)
    lib = _lib.gpu()
    ws_bytes = lib.mxq_gemm_workspace_bytes(batch, M, N, K, int(ae))    # few tiles: K is split
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=ac.device) if ws_bytes else None
    with torch.cuda.device(ac.device):
        rc = lib.mxq_gemm_mx_nt(ac.data_ptr(), asc.data_ptr(), int(ae), bc.data_ptr(),
                                bsc.data_ptr(), int(be), None if bias is None else bias.data_ptr(),
                                out.data_ptr(), _DTYPE[out_dtype], batch, M, N, K,
                                int(bool(epilogue_quant)), None if ws is None else ws.data_ptr(),
                                ws_bytes, _stream(ac))
    _lib.check(rc, lib)
    return out


def _use_nibbles(fa, fb, K):
    """Two fp4 operands go to the MFMA units as e2m1 nibbles (half the bytes, twice the rate)."""
    return fa == ElemFormat.fp4 and fb == ElemFormat.fp4 and K % (2 * GEMM_K_MULTIPLE) == 0


def pack_weight(w, a_fmt, w_fmt, mx_specs, round):
    """The packed form mx_gemm_nt would build for a (N, K) weight on every call, built once: (codes,
    scales, code kind) -- 1 byte per element (1/2 when both operand formats are fp4) plus 1/32 for
    the scales, against 2 for a bf16 weight -- or None when the fused GEMM would not take it."""
    fa, fb = _as_format(a_fmt), _as_format(w_fmt)
    if fa not in _PACKABLE or fb not in _PACKABLE:
        return None
    if mx_specs["block_size"] != 32 or mx_specs["shared_exp_method"] != "max":
        return None
    if round not in RoundingMode.string_enums() or not w.is_cuda or w.dtype not in _FUSED_DTYPES or w.dim() != 2:
        return None
    K = w.shape[-1]
    if K == 0 or K % GEMM_K_MULTIPLE != 0 or w.numel() == 0:
        return None
    scale_bits = mx_specs["scale_bits"] if mx_specs["scale_bits"] != 0 else 8
    return pack_mx(w.contiguous(), fb, scale_bits, round, mx_specs["mx_flush_fp32_subnorms"],
                   _use_nibbles(fa, fb, K), False)


def mx_gemm_nt(a, b_kmajor, a_fmt, b_fmt, mx_specs, round, bias=None, epilogue_quant=False,
               pre_bfloat16=False, packed_b=None):
    """a (..., M, K) x b_kmajor (N, K) or (..., N, K), both MX-quantized along K: the fused
    equivalent of quantize_mx_op(a, axes=[-1]) @ quantize_mx_op(b, axes=[-1]).T (+ bias, see
    gemm_nt).  pre_bfloat16 (a bool, or one per operand): the operand is a bf16 tensor that has not been
    through the layers' elementwise bfloat16 / round-half-away quantization yet; its pack kernel applies it.  Returns None
    when the operands do not qualify (the caller then takes the unfused path).  packed_b: what
    pack_weight returned for b_kmajor (a 2-D weight) under the same formats, specs and rounding; the
    pack of b is then skipped and b_kmajor is not looked at."""
    fa, fb = _as_format(a_fmt), _as_format(b_fmt)
    if fa not in _PACKABLE or fb not in _PACKABLE:
        return None
    if mx_specs["block_size"] != 32 or mx_specs["shared_exp_method"] != "max":
        return None
    if round not in RoundingMode.string_enums():
        return None
    if not a.is_cuda or a.dtype not in _FUSED_DTYPES or a.dim() < 2:
        return None
    K = a.shape[-1]
    if K == 0 or K % GEMM_K_MULTIPLE != 0 or a.numel() == 0:
        return None
    nibbles = _use_nibbles(fa, fb, K)
    if packed_b is not None:
        # a weight packed ahead of time: its codes and scales say what it is, b_kmajor is not read
        if packed_b[1].dim() != 2 or packed_b[1].shape[1] * 32 != K or \
                int(packed_b[2]) != _code_kind(fb, nibbles, "mx_gemm_nt"):
            raise RuntimeError("mx_gemm_nt: packed_b does not belong to these formats or this K")
        _packed_k(packed_b[0], packed_b[1], packed_b[2], "mx_gemm_nt")
        a2, b2 = a.contiguous().reshape(-1, K), None
        out_shape = a.shape[:-1] + (packed_b[1].shape[0],)
    else:
        if not b_kmajor.is_cuda or b_kmajor.dtype not in _FUSED_DTYPES or b_kmajor.dim() < 2 or \
                b_kmajor.shape[-1] != K or b_kmajor.numel() == 0:
            return None
        if b_kmajor.dim() == 2:
            a2 = a.contiguous().reshape(-1, K)              # fold every leading axis into M
            b2 = b_kmajor.contiguous()
            out_shape = a.shape[:-1] + (b2.shape[0],)
        elif b_kmajor.shape[:-2] == a.shape[:-2]:
            a2 = a.contiguous().reshape(-1, a.shape[-2], K)
            b2 = b_kmajor.contiguous().reshape(-1, b_kmajor.shape[-2], K)
            out_shape = a.shape[:-1] + (b_kmajor.shape[-2],)
            if a2.shape[0] > 65535:
                return None
        else:
            return None                                      # broadcast batch axes
    scale_bits = mx_specs["scale_bits"] if mx_specs["scale_bits"] != 0 else 8
    flush = mx_specs["mx_flush_fp32_subnorms"]
    if bias is not None and (bias.dtype != a.dtype or bias.dim() != 1):
        return None
    if epilogue_quant and a.dtype != torch.bfloat16:
        return None
    pre_a, pre_b = pre_bfloat16 if isinstance(pre_bfloat16, tuple) else (pre_bfloat16, pre_bfloat16)
    if (pre_a and a.dtype != torch.bfloat16) or (pre_b and b2 is not None and b2.dtype != torch.bfloat16):
        return None
    pa = pack_mx(a2, fa, scale_bits, round, flush, nibbles, pre_a)
    pb = packed_b if packed_b is not None else pack_mx(b2, fb, scale_bits, round, flush, nibbles, pre_b)
    return gemm_nt(pa, pb, out_dtype=a.dtype, bias=bias, epilogue_quant=epilogue_quant).reshape(out_shape)


SCORES_K, SCORES_MAX_N = 128, 2048


def mx_bmm_softmax(a, b_kmajor, fmt, mx_specs, round, exp2=False):
    """softmax(Q(a x b_kmajor^T), dim = -1) in one launch (include/mxq.h: mxq_bmm_softmax_mx_nt) for
    bf16 GPU operands a (..., M, 128), b_kmajor (..., N, 128) that have not been through the layers'
    elementwise bfloat16 quantization yet (the pack kernels apply it), N a multiple of 32 up to 2048,
    under the bfloat16 / round-half-away quantizer.  Returns None when the operands do not qualify."""
    f = _as_format(fmt)
    if f not in _PACKABLE or mx_specs["block_size"] != 32 or mx_specs["shared_exp_method"] != "max":
        return None
    if round not in RoundingMode.string_enums():
        return None
    if not (a.is_cuda and b_kmajor.is_cuda) or a.dtype != torch.bfloat16 or b_kmajor.dtype != torch.bfloat16:
        return None
    if a.dim() < 2 or a.dim() != b_kmajor.dim() or a.shape[:-2] != b_kmajor.shape[:-2]:
        return None
    K, M, N = a.shape[-1], a.shape[-2], b_kmajor.shape[-2]
    if K != SCORES_K or b_kmajor.shape[-1] != K or N == 0 or N % 32 != 0 or N > SCORES_MAX_N or M == 0:
        return None
    a3 = a.contiguous().reshape(-1, M, K)
    b3 = b_kmajor.contiguous().reshape(-1, N, K)
    batch = a3.shape[0]
    if batch == 0 or batch > 65535:
        return None
    scale_bits = mx_specs["scale_bits"] if mx_specs["scale_bits"] != 0 else 8
    flush = mx_specs["mx_flush_fp32_subnorms"]
    ac, asc, ak = pack_mx(a3, f, scale_bits, round, flush, False, True)
    bc, bsc, bk = pack_mx(b3, f, scale_bits, round, flush, False, True)
    out = torch.empty(a.shape[:-1] + (N,), dtype=torch.bfloat16, device=a.device)
    lib = _lib.gpu()
    with torch.cuda.device(a.device):
        rc = lib.mxq_bmm_softmax_mx_nt(ac.data_ptr(), asc.data_ptr(), int(ak), bc.data_ptr(), bsc.data_ptr(),
                                       int(bk), out.data_ptr(), batch, M, N, K, int(bool(exp2)),
                                       _flags_value(), _stream(a))
    _lib.check(rc, lib)
    return out


def mx_gemm_operands(operands, mx_specs, out_dtype):
    """General form of mx_gemm_nt for the gradient GEMMs: `operands` = two (tensor, format, round,
    transposed) entries.  transposed=False: the tensor is (..., rows, K), quantized along its last
    axis; True: it is (..., K, rows), quantized along its second-to-last axis and transposed while
    packing.  Returns rows_a x rows_b (leading axes must match, or the second operand has none),
    or None when the operands do not qualify."""
    if mx_specs["block_size"] != 32 or mx_specs["shared_exp_method"] != "max":
        return None
    packed, shapes = [], []
    for t, fmt, rnd, transposed in operands:
        f = _as_format(fmt)
        if f not in _PACKABLE or rnd not in RoundingMode.string_enums():
            return None
        if not t.is_cuda or t.dtype not in _FUSED_DTYPES or t.dim() < 2 or t.numel() == 0:
            return None
        K = t.shape[-2] if transposed else t.shape[-1]
        if K % GEMM_K_MULTIPLE != 0 or (transposed and t.shape[-1] % (8 // t.element_size()) != 0):
            return None
        shapes.append((t.shape[:-2], t.shape[-1] if transposed else t.shape[-2], K, transposed, f, rnd))
    (lead_a, rows_a, Ka, _, _, _), (lead_b, rows_b, Kb, _, _, _) = shapes
    if Ka != Kb or (len(lead_b) and lead_b != lead_a):
        return None
    if len(lead_a) and not len(lead_b) and operands[0][3]:
        return None                                   # a transposed batched A cannot be folded into rows
    scale_bits = mx_specs["scale_bits"] if mx_specs["scale_bits"] != 0 else 8
    flush = mx_specs["mx_flush_fp32_subnorms"]
    nibbles = _use_nibbles(shapes[0][4], shapes[1][4], Ka)
    for (t, _, _, _), (lead, rows, K, transposed, f, rnd) in zip(operands, shapes):
        t = t.contiguous()
        p = (pack_mx_t if transposed else pack_mx)(t, f, scale_bits, rnd, flush, nibbles)
        packed.append(p)
    (ac, asc, ae), (bc, bsc, be) = packed
    kb = Ka // 2 if nibbles else Ka                   # bytes of codes per row
    if len(lead_b):                                   # batched x batched
        batch = asc.numel() // (rows_a * (Ka // 32))
        if batch > 65535:
            return None
        ac, asc = ac.reshape(batch, rows_a, kb), asc.reshape(batch, rows_a, Ka // 32)
        bc, bsc = bc.reshape(batch, rows_b, kb), bsc.reshape(batch, rows_b, Ka // 32)
    else:                                             # every leading axis of A folds into its rows
        ac, asc = ac.reshape(-1, kb), asc.reshape(-1, Ka // 32)
    out = gemm_nt((ac, asc, ae), (bc, bsc, be), out_dtype=out_dtype)
    return out.reshape(tuple(lead_a) + (rows_a, rows_b))
