"""CPU oracle for the MX / bfloat quantization path.  TEST INFRASTRUCTURE ONLY.

This module restates, as a sequence of plain torch CPU tensor ops, the algorithm of the
reference's pure-PyTorch quantization path (``custom_cuda=False``).  It exists to check the
HIP kernels (tests, the smoke check and the ``cpu_baseline`` leg of the benchmark); no product
code may import it.

Why torch ops and not C or numpy: the reference's pure path *is* torch's CPU kernels
(``log2``, ``pow``, ``floor``, ``max``, ``clamp``, ``div``/``mul``) applied in the tensor's own dtype.
A bf16 tensor is rounded to bf16 after every op, and ``floor(log2(x))`` is evaluated in the
tensor dtype, so it returns k+1 for values just below 2**(k+1).  Both effects change output bits
and can only be restated faithfully by running the same ops, in the same order, in the same
dtype.  (A scalar C restatement of the same arithmetic lives in ``mxq_oracle.c``; the two are
checked against each other.)

Each function cites the reference lines it follows (paths relative to the reference root).

Parity status of every function here ("pinned" = checked against something other than itself):
  * format_params           pinned: closed-form constants of mx/tests/test_formats.py:12-95
  * quantize_elemwise_core  pinned for fp32 tensors: literal vectors of
                            mx/tests/test_quantize_elemwise.py:54-69 and
                            mx/tests/test_corners_elemwise.py (max/NaN/subnormal vectors), the
                            round='even' == ``x.to(bfloat16)`` / ``x.half()`` library special case,
                            idempotence on every encoding, and an exact-rational brute force.
                            bf16/fp16-dtype tensors and floor mode inside the log2 round-up
                            zone: pinned by golden fixtures written from the reference itself
                            (tests/golden/).
  * quantize_mx             pinned: literal vectors of mx/tests/test_fp8_e4m3_fix.py:17-18,92-108,
                            mx/tests/test_e5m0_scale.py:23-27, mx/tests/test_corners_mx.py:43-44,
                            62-67,84-112; exact-rational brute force; golden fixtures for bf16.
  * reduce_*_inner_dim      are torch.sum / torch.max themselves (the reference's own oracle,
                            mx/tests/test_reduce.py:17-20).
  * mx_linear_forward / _backward, mx_bmm_forward / _backward, softmax_forward / _backward
                            pinned (fp32 and bf16 tensors, bfloat 0 / 16, e^x and 2^x softmax):
                            forward outputs and gradients written by the reference's own layers on
                            the CPU (tests/golden/reference_layer_vectors.npz), reproduced bit for
                            bit (tests/test_layer_golden.py), including the vec_use_exp2 and
                            vec_use_recip switches and an fp= format of softmax_forward.
"""
import torch

ROUNDING_MODES = ("nearest", "floor", "even")          # mx/formats.py:12-19
_FP32_MIN_NORMAL = 2.0 ** -126                         # mx/formats.py:8-9
_FP32_EXP_BIAS = 127

# name -> (ebits, mbits); mbits counts sign + implicit one + trailing bits.  mx/formats.py:83-113
_FORMATS = {
    "int8": (0, 8), "int4": (0, 4), "int2": (0, 2),
    "fp8_e5m2": (5, 4), "fp8_e4m3": (4, 5),
    "fp6_e3m2": (3, 4), "fp6_e2m3": (2, 5),
    "fp4_e2m1": (2, 3), "fp4": (2, 3),
    "float16": (5, 12), "fp16": (5, 12),
    "bfloat16": (8, 9), "bf16": (8, 9),
}


def format_params(name):
    """(ebits, mbits, emax, max_norm, min_norm) of an element format.  mx/formats.py:61-125."""
    name = name.lower()
    ebits, mbits = _FORMATS[name]
    if ebits == 0:
        emax = 0
    elif ebits >= 5:                      # IEEE-like: top exponent reserved for Inf/NaN
        emax = 2 ** (ebits - 1) - 1
    else:                                 # OCP small floats use the top exponent for numbers
        emax = 2 ** (ebits - 1)
    if name == "fp8_e4m3":                # S.1111.111 is NaN, so the top mantissa is 1.75
        max_norm = 2 ** emax * 1.75
    else:
        max_norm = 2 ** emax * float(2 ** (mbits - 1) - 1) / 2 ** (mbits - 2)
    min_norm = 0 if ebits == 0 else 2 ** (2 - 2 ** (ebits - 1))
    return ebits, mbits, emax, max_norm, min_norm


def ieee_max_norm(ebits, mbits):
    """Largest normal of a format with Inf/NaN in the top exponent.  mx/formats.py:53-57."""
    emax = 2 ** (ebits - 1) - 1
    return 2 ** emax * float(2 ** (mbits - 1) - 1) / 2 ** (mbits - 2)


# ---------------------------------------------------------------------------------------------
# element rounding
# ---------------------------------------------------------------------------------------------
def _round_scaled(v, mode, noise=None):
    """Integer rounding of a pre-scaled tensor.  mx/elemwise_ops.py:45-76.  dither: `noise` stands in
    for the reference's torch.rand_like(v) so that a test can hand both sides the same draw."""
    if mode == "dither":
        rand = torch.rand_like(v, requires_grad=False) if noise is None else noise.reshape(v.shape)
        return torch.sign(v) * torch.floor(torch.abs(v) + rand)
    if mode == "floor":
        return torch.sign(v) * torch.floor(torch.abs(v))
    if mode == "nearest":
        return torch.sign(v) * torch.floor(torch.abs(v) + 0.5)
    if mode == "even":
        mag = torch.abs(v)
        is_tie_to_even = ((mag - 0.5) % 2 == torch.zeros_like(v)).type(v.dtype)
        return torch.sign(v) * (torch.floor(mag + 0.5) - is_tie_to_even)
    raise ValueError("unsupported rounding mode %r" % (mode,))


def quantize_elemwise_core(A, bits, exp_bits, max_norm, round="nearest",
                           saturate_normals=False, allow_denorm=True, noise=None):
    """Round every element of A to a (bits, exp_bits, max_norm) format.
    mx/elemwise_ops.py:82-170, pure branch (127-163)."""
    if not allow_denorm and exp_bits > 0:                                  # 128-130
        min_norm = 2 ** (2 - 2 ** (exp_bits - 1))
        out = (torch.abs(A) >= min_norm).type(A.dtype) * A
    else:
        out = A

    if exp_bits != 0:                                                      # 134-140
        private_exp = torch.floor(torch.log2(torch.abs(A) + (A == 0).type(A.dtype)))
        private_exp = private_exp.clip(min=2 - 2 ** (exp_bits - 1))
        out = out / (2 ** private_exp) * (2 ** (bits - 2))                 # 145, 31-35
    else:
        private_exp = None
        out = out * (2 ** (bits - 2))

    out = _round_scaled(out, round, noise)                                 # 147

    if private_exp is None:                                                # 150, 38-42
        out = out / (2 ** (bits - 2))
    else:
        out = out / (2 ** (bits - 2)) * (2 ** private_exp)

    if saturate_normals or exp_bits == 0:                                  # 153-157
        out = torch.clamp(out, min=-max_norm, max=max_norm)
    else:
        out = torch.where(torch.abs(out) > max_norm, torch.sign(out) * float("Inf"), out)

    out[A == float("Inf")] = float("Inf")                                  # 161-162
    out[A == -float("Inf")] = -float("Inf")
    return out


def quantize_bfloat(A, bfloat, round="nearest", allow_denorm=True):
    """bfloatX: 8 exponent bits, X-9 trailing bits.  mx/elemwise_ops.py:191-206."""
    if bfloat == 0 or bfloat == 32:
        return A
    return quantize_elemwise_core(A, bfloat - 7, 8, ieee_max_norm(8, bfloat - 7), round=round,
                                  allow_denorm=allow_denorm)


def quantize_fp(A, exp_bits, mantissa_bits, round="nearest", allow_denorm=True):
    """IEEE-like fpX.  mx/elemwise_ops.py:209-230."""
    if exp_bits is None or mantissa_bits is None:
        return A
    return quantize_elemwise_core(A, mantissa_bits + 2, exp_bits,
                                  ieee_max_norm(exp_bits, mantissa_bits + 2), round=round,
                                  allow_denorm=allow_denorm)


def quantize_elemwise_format(A, elem_format, round="nearest", saturate_normals=False,
                             allow_denorm=True):
    """mx/elemwise_ops.py:173-188."""
    if elem_format is None:
        return A
    ebits, mbits, _, max_norm, _ = format_params(elem_format)
    return quantize_elemwise_core(A, mbits, ebits, max_norm, round=round,
                                  saturate_normals=saturate_normals, allow_denorm=allow_denorm)


# ---------------------------------------------------------------------------------------------
# MX block quantization
# ---------------------------------------------------------------------------------------------
def shared_exponent(A, axes):
    """floor(log2(max |A| over axes)), keepdim, zero -> 2**-126.  mx/mx_ops.py:49-92 with
    method='max' and ebits=0 (the only way _quantize_mx calls it, mx/mx_ops.py:269-271)."""
    m = A
    for ax in axes:
        m, _ = torch.max(torch.abs(m), dim=ax, keepdim=True)
    return torch.floor(torch.log2(m + _FP32_MIN_NORMAL * (m == 0).type(m.dtype)))


def _to_blocks(A, axes, block_size):
    """Split every axis in `axes` into (n_blocks, block_size), zero padding a ragged tail.
    mx/mx_ops.py:95-154.  Returns the blocked view, the positions of the n_blocks axes, and the
    shapes needed to undo it."""
    axes = sorted(a + A.ndim if a < 0 else a for a in axes)
    for n, _ in enumerate(axes):
        axes[n] += n                       # every earlier split shifted this axis by one
        A = A.unsqueeze(axes[n] + 1)
    unpadded = list(A.shape)
    pad = []                               # F.pad wants (last_lo, last_hi, ..., first_lo, first_hi)
    for d in reversed(range(A.ndim)):
        extra = (-unpadded[d]) % block_size if d in axes else 0
        pad += [0, extra]
    if any(pad):
        A = torch.nn.functional.pad(A, pad, mode="constant")
    padded = list(A.shape)
    blocked = list(padded)
    for ax in axes:
        if blocked[ax] >= block_size:
            blocked[ax + 1] = block_size
            blocked[ax] //= block_size
        else:                               # short axis: one block of its own length
            blocked[ax + 1] = blocked[ax]
            blocked[ax] = 1
    return A.view(blocked), axes, unpadded, padded


def _from_blocks(A, axes, unpadded, padded):
    """mx/mx_ops.py:157-167."""
    A = A.view(padded)
    if padded != unpadded:
        A = A[tuple(slice(0, n) for n in unpadded)]
    for ax in reversed(axes):
        A = A.squeeze(ax + 1)
    return A


def quantize_mx(A, scale_bits, elem_format, axes, block_size=0, round="nearest",
                flush_fp32_subnorms=False, noise=None):
    """MX fake-quantization of A.  mx/mx_ops.py:173-298, pure branch (265-292),
    shared_exp_method='max'."""
    if elem_format is None:
        return A
    assert scale_bits > 0
    axes = [axes] if isinstance(axes, int) else list(axes)
    axes = [a + A.ndim if a < 0 else a for a in axes]
    ebits, mbits, emax, max_norm, _ = format_params(elem_format)

    if block_size > 0:
        A, axes, unpadded, padded = _to_blocks(A, axes, block_size)
        exp_axes = [a + 1 for a in axes]
    else:
        exp_axes = axes

    se = shared_exponent(A, exp_axes)                                      # 269-271
    if flush_fp32_subnorms:                                                # 274-275
        A = A * (se > -_FP32_EXP_BIAS).type(A.dtype)
    se = se - emax                                                         # 279
    scale_emax = 2 ** (scale_bits - 1) - 1                                 # 281-283
    se[se > scale_emax] = float("NaN")
    se[se < -scale_emax] = -scale_emax

    A = A / (2 ** se)                                                      # 285
    A = quantize_elemwise_core(A, mbits, ebits, max_norm, round=round,
                               allow_denorm=True, saturate_normals=True, noise=noise)   # 287-290
    A = A * (2 ** se)                                                      # 292

    if block_size > 0:
        A = _from_blocks(A, axes, unpadded, padded)
    return A


# ---------------------------------------------------------------------------------------------
# reductions: the reference checks its kernels against torch itself (mx/tests/test_reduce.py:17-20)
# ---------------------------------------------------------------------------------------------
def reduce_sum_inner_dim(A):
    return torch.sum(A, dim=-1)


def reduce_max_inner_dim(A):
    return torch.max(A, dim=-1).values


# ---------------------------------------------------------------------------------------------
# callers of the quantizer (forward only)
# ---------------------------------------------------------------------------------------------
def quantize_elemwise_op(A, bfloat=0, fp=0, round="nearest", bfloat_subnorms=True):
    """Spec plumbing of mx/elemwise_ops.py:233-267 (``A.to(bfloat16)`` shortcut at 248-251)."""
    if bfloat == 16 and round == "even" and bfloat_subnorms:
        return A.to(torch.bfloat16)
    if bfloat > 0 and fp > 0:
        raise ValueError("Cannot set both [bfloat] and [fp] in mx_specs.")
    if bfloat > 9:
        return quantize_bfloat(A, bfloat, round=round, allow_denorm=bfloat_subnorms)
    if bfloat > 0:
        raise ValueError("Cannot set [bfloat] <= 9 in mx_specs.")
    if fp > 6:
        return quantize_fp(A, 5, fp - 6, round=round, allow_denorm=bfloat_subnorms)
    if fp > 0:
        raise ValueError("Cannot set [fp] <= 6 in mx_specs.")
    return A


def mx_linear_forward(x, w, bias, w_fmt, a_fmt, block_size=32, scale_bits=8, bfloat=0,
                      round="nearest"):
    """Forward of the MX linear layer.  mx/linear.py:20-101: elementwise-quantize the operands,
    MX-quantize both along the contraction axis, fp32-accumulated matmul, elementwise-quantize,
    add the bias, elementwise-quantize."""
    q = lambda t: quantize_elemwise_op(t, bfloat=bfloat, round=round)
    bx, bw = q(x), q(w)
    qx = quantize_mx(bx, scale_bits, a_fmt, axes=[-1], block_size=block_size, round=round)
    qw = quantize_mx(bw, scale_bits, w_fmt, axes=[-1], block_size=block_size, round=round)
    out = q(torch.nn.functional.linear(qx, qw))
    if bias is not None:
        out = q(out + q(bias))
    return out


def mx_bmm_forward(a, b, fmt, block_size=32, scale_bits=8, bfloat=0, round="nearest"):
    """Forward of MX bmm.  mx/bmm.py:20-67: first operand shares exponents along its last axis,
    second along its second-to-last."""
    q = lambda t: quantize_elemwise_op(t, bfloat=bfloat, round=round)
    qa = quantize_mx(q(a), scale_bits, fmt, axes=[-1], block_size=block_size, round=round)
    qb = quantize_mx(q(b), scale_bits, fmt, axes=[-2], block_size=block_size, round=round)
    return q(torch.bmm(qa, qb))


def softmax_forward(x, dim, bfloat=16, round="nearest", use_exp2=False, vec_use_exp2=False,
                    vec_use_recip=False, fp=0):
    """Forward of the bfloat softmax chain.  mx/softmax.py:20-54 over mx/vector_ops.py:38-130:
    every step is a torch op followed by an elementwise quantization.  use_exp2 =
    mx_specs['softmax_exp2'] (softmax.py:35-37); vec_use_exp2 / vec_use_recip: vector_ops.py:73-77,
    59-62."""
    q = lambda t: quantize_elemwise_op(t, bfloat=bfloat, fp=fp, round=round)
    x = q(x)
    mx = torch.max(x, dim, keepdim=True).values
    x = q(x - mx)
    if use_exp2:
        e = q(torch.exp2(x))
    elif vec_use_exp2:
        e = q(torch.exp2(q(1.4453125 * x)))
    else:
        e = q(torch.exp(x))
    s = q(e.sum(dim, keepdim=True))
    if vec_use_recip:
        return q(e * q(1.0 / s))
    return q(e / s)


# ---- backward passes (mx_specs['quantize_backprop'] = True, one format / rounding throughout) ----
def mx_linear_backward(x, w, grad_out, has_bias, fmt, block_size=32, scale_bits=8, bfloat=0,
                       round="nearest"):
    """Backward of the MX linear layer.  mx/linear.py:103-198: the saved tensors are the
    elementwise-quantized input and weight (62-66); grad_weight contracts over the example axis
    (both operands MX-quantized along axis -2, 124-150), grad_input over the output features
    (weight along axis 0, grad_output along -1, 160-182), grad_bias is a plain sum (187-196).
    Returns (grad_input, grad_weight, grad_bias)."""
    q = lambda t: quantize_elemwise_op(t, bfloat=bfloat, round=round)
    mxq = lambda t, ax: quantize_mx(t, scale_bits, fmt, axes=[ax], block_size=block_size, round=round)
    bx, bw = q(x), q(w)
    out_dim, in_dim = w.shape
    go = q(grad_out)
    qex_in = mxq(bx, -2).reshape(-1, in_dim)
    qex_go = mxq(go, -2).reshape(-1, out_dim)
    grad_w = q(torch.matmul(qex_go.transpose(0, 1), qex_in))
    grad_in = q(torch.matmul(mxq(go, -1), mxq(bw, 0)))
    grad_b = q(go.reshape(-1, out_dim).sum(0)) if has_bias else None
    return grad_in, grad_w, grad_b


def mx_bmm_backward(a, b, grad_out, fmt, block_size=32, scale_bits=8, bfloat=0, round="nearest"):
    """Backward of MX bmm.  mx/bmm.py:69-127: in1 along -2 and in2 along -1 (the axes that are
    contracted now), grad_out once along -1 and once along -2.  Returns (grad_in1, grad_in2)."""
    q = lambda t: quantize_elemwise_op(t, bfloat=bfloat, round=round)
    mxq = lambda t, ax: quantize_mx(t, scale_bits, fmt, axes=[ax], block_size=block_size, round=round)
    ba, bb, go = q(a), q(b), q(grad_out)
    g1 = q(torch.bmm(mxq(go, -1), mxq(bb, -1).transpose(-1, -2)))
    g2 = q(torch.bmm(mxq(ba, -2).transpose(-1, -2), mxq(go, -2)))
    return g1, g2


def softmax_backward(out, grad_out, dim, bfloat=16, round="nearest", use_exp2=False):
    """Backward of the bfloat softmax.  mx/softmax.py:56-88: out * (g - sum(g * out)), every op
    followed by the elementwise quantizer; * ln2 at bfloat16 precision for the 2^x variant."""
    q = lambda t: quantize_elemwise_op(t, bfloat=bfloat, round=round)
    g = q(grad_out)
    dot = q(q(g * out).sum(dim, keepdim=True))
    gi = q(out * q(g - dot))
    if use_exp2:
        gi = q(gi * 0.69140625)
    return gi
