"""GPU parity: the HIP kernels, called through the C ABI, against the CPU oracle and the golden
fixtures.  Quantized outputs must match bit for bit (NaN payloads aside); reductions: max exact,
sum within 1e-5 * sum|x| of an fp64 sum."""
import numpy as np
import pytest
import torch

from helpers import assert_bits_equal, from_bits, golden
from oracle import mx_oracle as O

pytestmark = pytest.mark.gpu

MX_FORMATS = ["fp8_e4m3", "fp8_e5m2", "fp6_e3m2", "fp6_e2m3", "fp4_e2m1", "int8", "int4"]
ROUNDS = ["nearest", "floor", "even"]


@pytest.fixture(scope="module")
def dev():
    assert torch.cuda.is_available(), "these tests need a GPU"
    return torch.device("cuda:0")


def mx_gpu(x, *a, **k):
    from microxcaling_amd.mx_ops import _quantize_mx
    y = _quantize_mx(x, *a, **k)
    torch.cuda.synchronize()
    return y


def elem_gpu(x, *a, **k):
    from microxcaling_amd.elemwise_ops import _quantize_elemwise_core
    y = _quantize_elemwise_core(x, *a, **k)
    torch.cuda.synchronize()
    return y


def test_library_loads_on_gpu(dev):
    from microxcaling_amd import _lib
    assert _lib.gpu().mxq_version() >= 100


# ---- golden fixtures written from the reference's pure path -------------------------------------
@pytest.mark.parametrize("fmt", MX_FORMATS)
@pytest.mark.parametrize("rnd", ROUNDS)
def test_golden_mx_bf16_and_fp32_zone(dev, fmt, rnd):
    z, _ = golden()
    xb = from_bits(z["mx_bf16_x"], torch.bfloat16)
    y = mx_gpu(xb.to(dev), 8, fmt, axes=[-1], block_size=32, round=rnd)
    assert_bits_equal(y, from_bits(z["mx_bf16_y.%s.%s" % (fmt, rnd)], torch.bfloat16), "bf16")
    xz = from_bits(z["mx_fp32_zone_x"], torch.float32)
    y = mx_gpu(xz.to(dev), 8, fmt, axes=[-1], block_size=32, round=rnd)
    assert_bits_equal(y, from_bits(z["mx_fp32_zone_y.%s.%s" % (fmt, rnd)], torch.float32), "fp32")


def test_golden_mx_bf16_transposed_flush(dev):
    z, _ = golden()
    xb = from_bits(z["mx_bf16_x"], torch.bfloat16).t().contiguous()
    y = mx_gpu(xb.to(dev), 5, "fp8_e4m3", axes=[0], block_size=32, round="even",
               flush_fp32_subnorms=True)
    assert_bits_equal(y, from_bits(z["mx_bf16_y.t.fp8_e4m3.even.sb5.flush"], torch.bfloat16))


_ELEM_CFG = {"bf16": (9, 8, 2 ** 127 * 255 / 128), "fp16": (12, 5, 65504.0),
             "bf12": (5, 8, 2 ** 127 * 15 / 8), "e4m3": (5, 4, 448.0)}


def test_golden_elementwise(dev):
    z, _ = golden()
    xe = from_bits(z["elem_fp32_x"], torch.float32).to(dev)
    xb = from_bits(z["elem_bf16_x"], torch.bfloat16).to(dev)
    n = 0
    for k in z.files:
        if k.startswith("elem_fp32_y."):
            _, name, rnd, sat, den = k.split(".")
            b, e, m = _ELEM_CFG[name]
            y = elem_gpu(xe, b, e, m, round=rnd, saturate_normals=bool(int(sat)),
                         allow_denorm=bool(int(den)))
            assert_bits_equal(y, from_bits(z[k], torch.float32), k)
            n += 1
        elif k.startswith("elem_bf16_y."):
            _, name, rnd, sat = k.split(".")
            b, e, m = _ELEM_CFG[name]
            y = elem_gpu(xb, b, e, m, round=rnd, saturate_normals=bool(int(sat)))
            assert_bits_equal(y, from_bits(z[k], torch.bfloat16), k)
            n += 1
    assert n >= 15


# ---- seeded random inputs against the oracle ----------------------------------------------------
def test_config1_mxfp8_fp32_4096(dev):
    g = torch.Generator().manual_seed(0)
    x = torch.randn(4096, 4096, generator=g)
    want = O.quantize_mx(x, 8, "fp8_e4m3", axes=[-1], block_size=32, round="nearest")
    got = mx_gpu(x.to(dev), 8, "fp8_e4m3", axes=[-1], block_size=32, round="nearest")
    assert_bits_equal(got, want, "config 1")


def _outlier_bf16(rows, cols, seed):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(rows, cols, generator=g)
    idx = torch.randperm(cols, generator=g)[: max(1, cols // 100)]
    scale = torch.ones(cols)
    scale[idx] = torch.exp(2.0 * torch.randn(idx.numel(), generator=g))
    return (x * scale).to(torch.bfloat16)


@pytest.mark.parametrize("fmt", ["fp6_e3m2", "fp6_e2m3", "fp4_e2m1"])
@pytest.mark.parametrize("axis", [-1, -2])
@pytest.mark.parametrize("rnd", ROUNDS)
def test_config2_bf16_outliers(dev, fmt, axis, rnd):
    x = _outlier_bf16(2048, 2048, 7)
    want = O.quantize_mx(x, 8, fmt, axes=[axis], block_size=32, round=rnd)
    got = mx_gpu(x.to(dev), 8, fmt, axes=[axis], block_size=32, round=rnd)
    assert_bits_equal(got, want, "%s axis %d %s" % (fmt, axis, rnd))


def _wide_fp32(rows, cols, seed):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(rows, cols, generator=g, dtype=torch.float64)
    x = x * 10.0 ** (torch.rand(rows, cols, generator=g, dtype=torch.float64) * 80 - 40)
    x = x.to(torch.float32).reshape(-1)
    n = x.numel()
    sp = torch.randperm(n, generator=g)
    k = n // 1000
    x[sp[:k]] = torch.tensor([float("inf"), -float("inf"), float("nan")]).repeat(k // 3 + 1)[:k]
    m = n // 100
    sub = torch.randint(1, 1 << 23, (m,), generator=g, dtype=torch.int32)
    sub |= torch.randint(0, 2, (m,), generator=g, dtype=torch.int32) << 31
    x[sp[k:k + m]] = sub.view(torch.float32)
    return x.reshape(rows, cols)


@pytest.mark.parametrize("bits,ebits,max_norm", [(9, 8, 2 ** 127 * 255 / 128), (12, 5, 65504.0)])
@pytest.mark.parametrize("rnd", ROUNDS)
@pytest.mark.parametrize("sat", [False, True])
def test_config3_elementwise(dev, bits, ebits, max_norm, rnd, sat):
    x = _wide_fp32(2048, 1024, 11)
    want = O.quantize_elemwise_core(x.clone(), bits, ebits, max_norm, round=rnd,
                                    saturate_normals=sat)
    got = elem_gpu(x.to(dev), bits, ebits, max_norm, round=rnd, saturate_normals=sat)
    assert_bits_equal(got, want, "elementwise")


def _sum_case(seed):
    """Wide-range finite values (|x| <= 1e30 so fp32 partial sums cannot overflow) with 0.1 % of
    the entries set to +Inf / -Inf / NaN: some rows stay finite, others must come out Inf or NaN."""
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(2048, 1024, generator=g) * 10.0 ** (torch.rand(2048, 1024, generator=g) * 60 - 30)
    pos = torch.randperm(x.numel(), generator=g)[: x.numel() // 1000]
    x.view(-1)[pos] = torch.tensor([float("inf"), -float("inf"), float("nan")]).repeat(
        pos.numel() // 3 + 1)[: pos.numel()]
    return x


def check_sum(got, x, dim):
    got = got.cpu().double()
    ref = x.double().sum(dim)                          # Inf / NaN class as IEEE addition gives it
    assert torch.equal(torch.isnan(got), torch.isnan(ref))
    inf = torch.isinf(ref)
    assert inf.any() and torch.equal(got[inf], ref[inf])
    fin = torch.isfinite(ref)
    assert fin.sum() >= 4
    tol = 1e-5 * torch.where(torch.isfinite(x), x, torch.zeros_like(x)).double().abs().sum(dim)
    assert ((got[fin] - ref[fin]).abs() <= tol[fin]).all()


def test_config3_reductions(dev):
    from microxcaling_amd.custom_extensions import funcs
    x = _sum_case(13)
    xd = x.to(dev)
    check_sum(funcs.reduce_sum_inner_dim(xd), x, -1)
    x = x.t().contiguous()                             # axis 0: 1024 x 2048, specials per column
    check_sum(funcs.reduce_sum_outer_dim(x.to(dev)), x, 0)
    y = _wide_fp32(2048, 1024, 17)                    # max: exact, NaN propagates like torch.max
    yd = y.to(dev)
    assert_bits_equal(funcs.reduce_max_inner_dim(yd), torch.max(y, dim=-1).values, "max -1")
    assert_bits_equal(funcs.reduce_max_outer_dim(yd), torch.max(y, dim=0).values, "max 0")
    y[torch.isnan(y)] = 0.5                           # and without NaNs
    yd = y.to(dev)
    assert_bits_equal(funcs.reduce_max_inner_dim(yd), torch.max(y, dim=-1).values, "max -1")
    assert_bits_equal(funcs.reduce_max_outer_dim(yd), torch.max(y, dim=0).values, "max 0")


@pytest.mark.parametrize("S,H", [(5, 32), (35, 32), (7, 512), (3, 1024), (15, 2048), (11, 4096),
                                 (3, 100)])
def test_reduce_reference_shapes(dev, S, H):
    """Shapes of the reference's own reduce test (mx/tests/test_reduce.py:21-28, tol 1e-6 RMS)."""
    from microxcaling_amd.custom_extensions import funcs
    g = torch.Generator().manual_seed(S * 1000 + H)
    m = torch.randn(64, S, H, generator=g)
    md = m.to(dev)
    s = funcs.reduce_sum_inner_dim(md).cpu()
    ref = m.sum(-1)
    assert (s - ref).abs().max() <= 1e-6 * (1 + ref.pow(2).mean().sqrt()) * 4
    assert_bits_equal(funcs.reduce_max_inner_dim(md), m.max(-1).values, "max")


# ---- shapes: axes, ragged blocks, other block sizes, empty --------------------------------------
@pytest.mark.parametrize("shape,axis,bs", [
    ((3, 70, 5), 1, 32), ((3, 70, 8), 1, 32), ((4, 64), 0, 32), ((130, 48), 0, 32),
    ((7, 96), 1, 8), ((7, 90), 1, 9), ((5, 128), 1, 64), ((5, 100), 1, 64), ((2, 3, 64), 2, 16),
    ((2, 40, 3, 4), 1, 32), ((6, 33), 1, 0), ((9, 256), 1, 128), ((9, 64), 1, 4), ((65, 7), 0, 10),
])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_mx_shapes(dev, shape, axis, bs, dtype):
    g = torch.Generator().manual_seed(sum(shape) + bs)
    x = (torch.randn(*shape, generator=g) * torch.exp(torch.randn(*shape, generator=g))).to(dtype)
    for fmt, rnd in (("fp8_e4m3", "nearest"), ("fp4_e2m1", "even"), ("int8", "floor")):
        want = O.quantize_mx(x, 8, fmt, axes=[axis], block_size=bs, round=rnd)
        got = mx_gpu(x.to(dev), 8, fmt, axes=[axis], block_size=bs, round=rnd)
        assert_bits_equal(got, want, "%s %s %s" % (shape, fmt, rnd))


@pytest.mark.parametrize("dt", ["f32", "bf16"])
@pytest.mark.parametrize("fmt", ["fp8_e4m3", "fp6_e2m3", "fp4_e2m1", "int8"])
def test_an_exponent_per_element_on_the_gpu(dev, fmt, dt):
    """shared_exp_method="none" (mx/mx_ops.py:49-92 with method "none") = blocks of one element, against
    what the reference returned (tests/golden/gen_reference_layer_vectors.py)."""
    import numpy as np
    import os
    from helpers import ROOT_DIR
    from microxcaling_amd.mx_ops import quantize_mx_op
    from microxcaling_amd.specs import finalize_mx_specs
    fix = np.load(os.path.join(ROOT_DIR, "tests", "golden", "reference_layer_vectors.npz"))
    qa = torch.from_numpy(fix["in/qa:f32"].copy()).view(torch.float32)
    tdt = torch.float32 if dt == "f32" else torch.bfloat16
    for block in (32, 0):
        specs = finalize_mx_specs(dict(a_elem_format=fmt, w_elem_format=fmt, block_size=block,
                                       shared_exp_method="none"))
        for ax in (-1, 0):
            key = "mx_none/%s/block%d/%s/axis%d:%s" % (fmt, block, dt, ax, dt)
            want = torch.from_numpy(fix[key].copy()).view(tdt)
            got = quantize_mx_op(qa.to(tdt).to(dev), specs, elem_format=fmt, axes=[ax], round="nearest")
            assert_bits_equal(got.cpu(), want, key)


@pytest.mark.parametrize("shape,axes,bs", [((70, 45), [-2, -1], 32), ((3, 40, 5, 33), [1, 3], 8),
                                           ((6, 10, 12), [0, 1, 2], 4), ((5, 64, 64), [1, 2], 0),
                                           ((4, 7, 9), [2, 0], 32), ((2, 3, 4, 5, 6), [1, 2, 4], 2),
                                           ((256, 384), [0, 1], 32), ((3, 100, 300), [1, 2], 64),
                                           ((3, 64, 96), [1, 2], 32), ((2, 5, 32, 32), [-2, -1], 32),
                                           ((64, 96, 2), [0, 1], 32)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_mx_several_axes(dev, shape, axes, bs, dtype):
    """One exponent per tile of bs x bs (x bs) elements over two or three axes (mx/mx_ops.py:95-154,
    226-298 with len(axes) > 1), against the oracle's restatement of the pure path."""
    g = torch.Generator().manual_seed(sum(shape) + bs)
    x = (torch.randn(*shape, generator=g) * torch.exp2(torch.randint(-12, 12, shape, generator=g).float())).to(dtype)
    x.view(-1)[3] = 0.0
    x.view(-1)[-1] = float("nan")
    for fmt, rnd in (("fp8_e4m3", "nearest"), ("fp6_e3m2", "floor"), ("fp4_e2m1", "even"), ("int8", "nearest")):
        want = O.quantize_mx(x, 8, fmt, axes=axes, block_size=bs, round=rnd)
        got = mx_gpu(x.to(dev), 8, fmt, axes=axes, block_size=bs, round=rnd)
        assert_bits_equal(got, want, "%s %s %s" % (shape, fmt, rnd))


def test_dither_with_the_reference_noise(dev):
    """round='dither' on the GPU with the noise the reference drew (torch.rand_like under the stored
    seed, regenerated on the CPU and copied over): the reference's outputs bit for bit."""
    from helpers import dither_cases, reference_noise
    from microxcaling_amd.custom_extensions import funcs
    from microxcaling_amd.formats import _get_format_params
    for kind, name, dtype, case_no, seed, case, x, want in dither_cases():
        if dtype == torch.float16:
            continue                                  # tests/test_zx_fp16_tensors.py
        if kind == "mx" and case[2] > 0 and x.shape[case[1]] % case[2] != 0:
            continue                                  # ragged blocks: tests/test_zt_uncommon_parameters.py
        torch.manual_seed(seed)
        noise = reference_noise(kind, case, x).to(dev)
        if kind == "mx":
            fmt, axis, bs = case
            ebits, mbits, _, max_norm, _ = _get_format_params(fmt)
            got = funcs.quantize_mx_dither_by_tile_func(x.to(dev), noise, 8, ebits, mbits, max_norm, bs,
                                                        axis % x.ndim, False)
        else:
            bits, eb, mn, sat = case
            got = funcs.quantize_elemwise_dither_func(x.to(dev), noise, bits, eb, mn, sat, True)
        torch.cuda.synchronize()
        assert_bits_equal(got, want, "%s %s %d" % (kind, name, case_no))
    # through the public call: the noise comes from torch's generator for the device
    xs = torch.linspace(-3.9, 3.9, 4001, device=dev)
    from microxcaling_amd.elemwise_ops import _quantize_elemwise_core
    draws = torch.stack([_quantize_elemwise_core(xs, 5, 4, 448.0, round="dither") for _ in range(200)])
    lo = _quantize_elemwise_core(xs, 5, 4, 448.0, round="floor")
    step = torch.exp2(torch.floor(torch.log2(xs.abs().clamp_min(2.0 ** -6))) - 3)
    assert ((draws == lo) | (draws == lo + torch.sign(xs) * step)).all()
    assert ((draws.mean(0) - xs).abs() <= 0.3 * step).all()
    got = mx_gpu(torch.randn(64, 64, device=dev), 8, "fp4_e2m1", axes=[-1], block_size=32, round="dither")
    assert torch.isfinite(got).all()


def test_bf16_to_bfloat16_closed_form_every_code(dev):
    """bf16 tensors quantized to bfloat16 with round-half-away take a kernel of their own (closed
    form, packed pairs in the plain range): every bf16 code, in waves of plain values only and in
    mixed order, with a ragged tail, against the oracle."""
    codes = torch.arange(0, 65536, dtype=torch.int32).to(torch.int16).view(torch.bfloat16)
    mags = codes.float().abs()
    plain = codes[(mags >= 2.0 ** -126) & (mags < 2.0 ** 127)]
    g = torch.Generator().manual_seed(21)
    x = torch.cat([plain.repeat(4), codes[torch.randperm(65536, generator=g)], codes, plain[:4099]])
    mn = 2 ** 127 * 255 / 128
    want = O.quantize_elemwise_core(x, 9, 8, mn, round="nearest")
    got = elem_gpu(x.to(dev), 9, 8, mn, round="nearest")
    assert_bits_equal(got, want, "closed form")
    # the neighbouring cases stay on the general kernel and agree with the oracle as before
    for kw in (dict(round="floor"), dict(round="nearest", saturate_normals=True), dict(round="nearest", allow_denorm=False)):
        assert_bits_equal(elem_gpu(x.to(dev), 9, 8, mn, **kw), O.quantize_elemwise_core(x, 9, 8, mn, **kw), str(kw))


def test_mx_given_max_entry_point(dev):
    """quantize_mx_func_cuda: the caller reshapes to blocks and supplies the abs-max
    (mx/mx_ops.py:226-256)."""
    from microxcaling_amd.custom_extensions import funcs
    from microxcaling_amd.formats import _get_format_params
    g = torch.Generator().manual_seed(5)
    for dtype in (torch.float32, torch.bfloat16):
        x = torch.randn(16, 4, 64, generator=g).to(dtype)
        want = O.quantize_mx(x.reshape(16, 256), 8, "fp8_e5m2", axes=[-1], block_size=64,
                             round="even").reshape(16, 4, 64)
        xd = x.to(dev)
        mv = xd.abs().max(dim=2, keepdim=True).values
        ebits, mbits, _, max_norm, _ = _get_format_params("fp8_e5m2")
        got = funcs.quantize_mx_func_cuda(xd, 8, ebits, mbits, max_norm, mv, 2, False, 2)
        assert_bits_equal(got, want, "given max")


def test_empty_inputs(dev):
    x = torch.zeros(0, dtype=torch.float32, device=dev)
    assert mx_gpu(x, 8, "fp8_e4m3", axes=[-1], block_size=32).numel() == 0
    assert elem_gpu(x, 9, 8, 3e38).numel() == 0


def test_errors_are_raised(dev):
    from microxcaling_amd.custom_extensions import funcs
    x = torch.zeros(4, 4, device=dev)
    with pytest.raises(RuntimeError):
        funcs.quantize_mx_by_tile_func_cuda(x.t(), 8, 4, 5, 448.0, 32, 1)      # not contiguous
    with pytest.raises(RuntimeError):
        funcs.quantize_mx_by_tile_func_cuda(x.cpu(), 8, 4, 5, 448.0, 32, 1)    # not on the GPU
    with pytest.raises(RuntimeError):
        funcs.quantize_mx_by_tile_func_cuda(x, 8, 4, 5, 448.0, 32, 2)          # axis out of range
    with pytest.raises(RuntimeError):
        funcs.quantize_elemwise_func_cuda(x, 30, 8, 3e38)                      # bits > 24
    with pytest.raises(RuntimeError):
        funcs.quantize_elemwise_func_cuda(x.double(), 9, 8, 3e38)              # dtype


# ---- full-size properties ------------------------------------------------------------------------
def test_headline_size_properties(dev):
    """8192 x 8192 fp32 MXFP8: idempotence, sign symmetry, agreement of the last-axis kernel with
    the strided kernel on the transposed tensor, and a block-sampled comparison with the oracle."""
    g = torch.Generator().manual_seed(0)
    x = torch.randn(8192, 8192, generator=g)
    xd = x.to(dev)
    y = mx_gpu(xd, 8, "fp8_e4m3", axes=[-1], block_size=32)
    assert torch.equal(mx_gpu(y, 8, "fp8_e4m3", axes=[-1], block_size=32), y)
    assert torch.equal(mx_gpu(-xd, 8, "fp8_e4m3", axes=[-1], block_size=32), -y)
    yt = mx_gpu(xd.t().contiguous(), 8, "fp8_e4m3", axes=[0], block_size=32)
    assert torch.equal(yt.t(), y)
    rows = torch.randperm(8192, generator=g)[:128]
    want = O.quantize_mx(x[rows], 8, "fp8_e4m3", axes=[-1], block_size=32)
    assert_bits_equal(y[rows.to(dev)], want, "sampled rows")
