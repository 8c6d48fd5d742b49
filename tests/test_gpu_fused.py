"""GPU tests of the packed MX form and the scaled-MFMA GEMM, and of the layers built on them."""
import pytest
import torch

from helpers import assert_bits_equal
from oracle import mx_oracle as O

pytestmark = pytest.mark.gpu


@pytest.fixture(autouse=True)
def products_evaluated_at_once():
    """mx.bmm as a kernel of its own in this file: the tests here compare the separate kernels with each other
    and with mx.bmm_softmax (the deferred product of mx.bmm has tests/test_zv_deferred_product_gpu.py)."""
    from microxcaling_amd import gemm
    gemm.set_deferred_scores(False)
    yield
    gemm.set_deferred_scores(True)
PACKABLE = ["fp8_e4m3", "fp8_e5m2", "fp6_e3m2", "fp6_e2m3", "fp4_e2m1"]


@pytest.fixture(scope="module")
def dev():
    assert torch.cuda.is_available()
    return torch.device("cuda:0")


def rel_err(got, want):
    got, want = got.double().cpu(), want.double().cpu()
    return ((got - want).abs().max() / want.pow(2).mean().sqrt()).item()


@pytest.mark.parametrize("fmt", PACKABLE)
@pytest.mark.parametrize("rnd", ["nearest", "floor", "even"])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_pack_then_unpack_is_the_fake_quantized_tensor(dev, fmt, rnd, dtype):
    """codes x 2^(scale-127) must be bit-identical to the oracle's _quantize_mx output, including
    subnormal blocks, -0.0 and NaN blocks."""
    from microxcaling_amd.fused import pack_mx, unpack_mx
    g = torch.Generator().manual_seed(21)
    x = torch.randn(96, 256, generator=g) * torch.exp(3 * torch.randn(96, 256, generator=g))
    x[3, 40] = float("inf")
    x[5, 70] = float("nan")
    x[7, :64] *= 1e-38
    x[9, :32] = 0.0
    x[11, :32] = -1e-30 * torch.rand(32, generator=g)
    x = x.to(dtype)
    want = O.quantize_mx(x, 8, fmt, axes=[-1], block_size=32, round=rnd)
    codes, scales, e5m2 = pack_mx(x.to(dev), fmt, 8, rnd)
    assert codes.shape == x.shape and scales.shape == (96, 8) and e5m2 == (fmt == "fp8_e5m2")
    got = unpack_mx(codes, scales, e5m2, dtype)
    torch.cuda.synchronize()
    assert_bits_equal(got, want, fmt)


@pytest.mark.parametrize("M,N,K,batch", [(128, 128, 128, 1), (256, 384, 512, 1), (100, 72, 256, 1),
                                         (130, 257, 128, 3), (16, 16, 128, 2), (1, 5, 384, 1),
                                         (512, 768, 256, 1), (600, 520, 128, 2),
                                         # large shapes with few tiles: small tiles, K split
                                         (512, 768, 512, 1), (600, 520, 1024, 2), (1024, 512, 2048, 1),
                                         (600, 520, 640, 2), (1024, 768, 1152, 1), (512, 512, 896, 1),
                                         # the persistent 256 x 256 kernel (at least 128 tiles): fewer
                                         # tiles than CUs, several tiles per workgroup, ragged edges
                                         (2048, 2048, 512, 2), (2048, 2048, 512, 5), (2050, 1800, 1024, 5),
                                         (4096, 2048, 1024, 1), (530, 512, 512, 22),
                                         # ... with a partial last scale group (K % 512 != 0)
                                         (2050, 1800, 1408, 3), (2048, 4096, 640, 1), (1100, 1500, 1152, 5),
                                         # few output tiles: K split over several workgroups per tile
                                         (64, 1024, 2048, 1), (16, 2050, 4096, 2), (100, 520, 1152, 1),
                                         (1, 128, 8192, 1)])
@pytest.mark.parametrize("fa,fb", [("fp8_e4m3", "fp8_e4m3"), ("fp8_e5m2", "fp8_e4m3"),
                                   ("fp6_e2m3", "fp8_e5m2"), ("fp4_e2m1", "fp6_e3m2")])
def test_scaled_mfma_gemm_against_fp64(dev, M, N, K, batch, fa, fb):
    """Per-block scale spread of 2^-3 .. 2^3 so that a wrong lane-to-scale mapping cannot hide.
    Tolerance 1e-3 (max |diff| / RMS): one scaled MFMA keeps about 14 bits relative to the sum of
    the magnitudes of the 128 products it adds, measured 7e-5 at worst."""
    from microxcaling_amd.fused import pack_mx, unpack_mx, gemm_nt
    g = torch.Generator().manual_seed(M * 7 + N * 3 + K + batch)
    shape_a = (batch, M, K) if batch > 1 else (M, K)
    shape_b = (batch, N, K) if batch > 1 else (N, K)
    blk = lambda s: torch.exp2(torch.randint(-3, 4, s[:-1] + (s[-1] // 32, 1), generator=g).float())
    a = (torch.randn(*shape_a, generator=g).view(*shape_a[:-1], K // 32, 32) * blk(shape_a)).view(shape_a)
    b = (torch.randn(*shape_b, generator=g).view(*shape_b[:-1], K // 32, 32) * blk(shape_b)).view(shape_b)
    pa = pack_mx(a.to(dev), fa)
    pb = pack_mx(b.to(dev), fb)
    got = gemm_nt(pa, pb, torch.float32)
    qa = unpack_mx(*pa, torch.float32).double()
    qb = unpack_mx(*pb, torch.float32).double()
    want = qa @ qb.transpose(-1, -2)
    torch.cuda.synchronize()
    assert got.shape == want.shape
    assert rel_err(got, want) < 1e-3
    den = qa.abs() @ qb.abs().transpose(-1, -2)
    assert ((got.double() - want).abs() <= 2e-4 * den + 1e-30).all()


@pytest.mark.parametrize("M,N,K,batch", [(128, 136, 256, 1), (600, 520, 1024, 2), (1024, 512, 2048, 1),
                                         (2050, 1800, 512, 5), (520, 777, 512, 1), (1030, 520, 1152, 2),
                                         (64, 1032, 2048, 1), (30, 777, 1024, 2), (2050, 1800, 1152, 2),
                                         (2048, 4104, 512, 1)])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("with_bias", [False, True])
def test_gemm_16bit_outputs_equal_rounded_fp32_output(dev, M, N, K, batch, dtype, with_bias):
    """The accumulation does not depend on the output type, so a 16-bit output must be the fp32
    output rounded once (and, with a bias, rounded, added to and rounded again), bit for bit --
    whatever layout the kernel chooses for the output type."""
    from microxcaling_amd.fused import pack_mx, gemm_nt
    g = torch.Generator().manual_seed(M + N + K + batch)
    sa = (batch, M, K) if batch > 1 else (M, K)
    sb = (batch, N, K) if batch > 1 else (N, K)
    pa = pack_mx(torch.randn(*sa, generator=g).to(dev), "fp8_e4m3")
    pb = pack_mx(torch.randn(*sb, generator=g).to(dev), "fp8_e5m2")
    bias = torch.randn(N, generator=g).to(dev).to(dtype) if with_bias else None
    want = gemm_nt(pa, pb, torch.float32).to(dtype)
    if with_bias:
        want = want + bias
    got = gemm_nt(pa, pb, dtype, bias=bias)
    torch.cuda.synchronize()
    assert got.dtype == dtype and torch.equal(got.view(torch.int16), want.view(torch.int16))


@pytest.mark.parametrize("M,N,K,batch", [(128, 136, 256, 1), (600, 520, 1024, 2), (2050, 1800, 512, 3),
                                         (64, 1032, 2048, 1)])
@pytest.mark.parametrize("with_bias", [False, True])
def test_gemm_epilogue_quantization_equals_separate_steps(dev, M, N, K, batch, with_bias):
    """epilogue_quant: the bfloat16 / round-half-away quantization after the product and after the
    bias add, done inside the GEMM, against the same steps done with the elementwise kernel
    (itself bit-identical to the oracle) on the fp32 product -- bit for bit."""
    from microxcaling_amd.fused import pack_mx, gemm_nt
    from microxcaling_amd.elemwise_ops import _quantize_bfloat
    g = torch.Generator().manual_seed(M + N + K + batch + 1)
    sa = (batch, M, K) if batch > 1 else (M, K)
    sb = (batch, N, K) if batch > 1 else (N, K)
    pa = pack_mx((torch.randn(*sa, generator=g) * 7).to(dev), "fp8_e4m3")
    pb = pack_mx(torch.randn(*sb, generator=g).to(dev), "fp6_e2m3")
    bias = torch.randn(N, generator=g).to(dev).to(torch.bfloat16) if with_bias else None
    want = _quantize_bfloat(gemm_nt(pa, pb, torch.float32).to(torch.bfloat16), 16, round="nearest")
    if with_bias:
        want = _quantize_bfloat(want + bias, 16, round="nearest")
    got = gemm_nt(pa, pb, torch.bfloat16, bias=bias, epilogue_quant=True)
    torch.cuda.synchronize()
    assert torch.equal(got.view(torch.int16), want.view(torch.int16))
    # the quantizer is not the identity on bf16: about half of the values must have moved
    plain = gemm_nt(pa, pb, torch.bfloat16, bias=bias)
    assert (plain != got).float().mean().item() > 0.2


@pytest.mark.parametrize("fmt", PACKABLE)
@pytest.mark.parametrize("rnd", ["nearest", "floor", "even"])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("shape", [(64, 40), (3, 96, 264), (128, 8), (160, 1032), (2, 288, 520), (1024, 64)])
def test_transposing_pack_equals_axis_minus2_quantization(dev, fmt, rnd, dtype, shape):
    """pack_mx_t = quantize along the second-to-last axis, transposed: bit for bit, including
    blocks with zeros, subnormals and NaN."""
    from microxcaling_amd.fused import pack_mx_t, unpack_mx
    from microxcaling_amd.mx_ops import _quantize_mx
    g = torch.Generator().manual_seed(sum(shape))
    x = (torch.randn(*shape, generator=g) * torch.exp2(torch.randint(-20, 20, shape[:-2] + (1, shape[-1]), generator=g).float())).to(dtype)
    x[..., 0:32, 1] = 0.0
    x[..., 32:64, 2] = 1e-39 if dtype == torch.float32 else 1e-38
    x[..., 5, 3] = float("nan")
    xd = x.to(dev)
    codes, scales, e5m2 = pack_mx_t(xd, fmt, round=rnd)
    assert codes.shape == shape[:-2] + (shape[-1], shape[-2]) and scales.shape == shape[:-2] + (shape[-1], shape[-2] // 32)
    got = unpack_mx(codes, scales, e5m2, dtype).transpose(-1, -2)
    want = _quantize_mx(xd, 8, fmt, axes=[-2], block_size=32, round=rnd)
    assert_bits_equal(got.contiguous().cpu(), want.cpu(), "pack_mx_t")


@pytest.mark.parametrize("rnd", ["nearest", "floor", "even"])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_nibble_pack_is_the_fake_quantized_tensor(dev, rnd, dtype):
    """fp4 elements as e2m1 nibbles (two per byte): unpacking gives the oracle's _quantize_mx output
    bit for bit, for the row-wise and for the transposing pack; the low nibble is the lower index."""
    from microxcaling_amd.fused import pack_mx, pack_mx_t, unpack_mx, CODES_E2M1
    g = torch.Generator().manual_seed(77)
    x = torch.randn(96, 256, generator=g) * torch.exp(3 * torch.randn(96, 256, generator=g))
    x[3, 40] = float("inf")
    x[5, 70] = float("nan")
    x[7, :64] *= 1e-38
    x[9, :32] = 0.0
    x[11, :32] = -1e-30 * torch.rand(32, generator=g)
    x = x.to(dtype)
    want = O.quantize_mx(x, 8, "fp4_e2m1", axes=[-1], block_size=32, round=rnd)
    codes, scales, kind = pack_mx(x.to(dev), "fp4_e2m1", 8, rnd, nibbles=True)
    assert codes.shape == (96, 128) and scales.shape == (96, 8) and kind == CODES_E2M1
    assert_bits_equal(unpack_mx(codes, scales, kind, dtype), want, "nibbles")
    # same values as the byte codes, element 2i in the low nibble of byte i
    bytes_, scales8, kind8 = pack_mx(x.to(dev), "fp4_e2m1", 8, rnd)
    assert torch.equal(scales8, scales)
    lut = torch.tensor([0, .5, 1, 1.5, 2, 3, 4, 6, -0., -.5, -1, -1.5, -2, -3, -4, -6], device=dev)
    ones = torch.full_like(scales8, 127)
    lo, hi = lut[(codes & 15).long()], lut[(codes >> 4).long()]
    elems = unpack_mx(bytes_, ones, kind8, torch.float32)
    finite = (scales8 != 255).repeat_interleave(32, dim=-1)
    assert torch.equal(torch.stack([lo, hi], -1).reshape(96, 256)[finite], elems[finite])
    # transposing pack
    want_t = O.quantize_mx(x, 8, "fp4_e2m1", axes=[-2], block_size=32, round=rnd)
    codes, scales, kind = pack_mx_t(x.to(dev), "fp4_e2m1", 8, rnd, nibbles=True)
    assert codes.shape == (256, 48) and scales.shape == (256, 3) and kind == CODES_E2M1
    got = unpack_mx(codes, scales, kind, dtype).transpose(-1, -2).contiguous()
    assert_bits_equal(got, want_t, "nibbles, transposed")
    with pytest.raises(RuntimeError, match="nibbles"):
        pack_mx(x.to(dev), "fp8_e4m3", nibbles=True)


@pytest.mark.parametrize("M,N,K,batch", [(128, 128, 256, 1), (100, 72, 256, 1), (130, 257, 768, 3),
                                         (1, 5, 512, 1), (600, 520, 256, 2),
                                         # persistent kernel (K % 512 == 0)
                                         (512, 768, 512, 1), (600, 520, 1024, 2), (1024, 512, 2048, 1),
                                         (2050, 1800, 1536, 3),
                                         # ... with a partial last scale group (K % 512 != 0)
                                         (600, 520, 768, 2), (1024, 768, 1280, 1), (2050, 1800, 2304, 2),
                                         # few output tiles: K split over several workgroups per tile
                                         (64, 1024, 2048, 1), (16, 2050, 4096, 2)])
def test_fp4_gemm_on_nibbles_against_fp64(dev, M, N, K, batch):
    """Both operands as e2m1 nibbles at the 4-bit MFMA rate: against fp64 on the unpacked operands,
    with a 2^-3 .. 2^3 spread of block scales, and against the same GEMM on byte codes (same
    products; only the grouping of the additions differs)."""
    from microxcaling_amd.fused import pack_mx, unpack_mx, gemm_nt
    g = torch.Generator().manual_seed(M * 7 + N * 3 + K + batch)
    shape_a = (batch, M, K) if batch > 1 else (M, K)
    shape_b = (batch, N, K) if batch > 1 else (N, K)
    blk = lambda s: torch.exp2(torch.randint(-3, 4, s[:-1] + (s[-1] // 32, 1), generator=g).float())
    a = (torch.randn(*shape_a, generator=g).view(*shape_a[:-1], K // 32, 32) * blk(shape_a)).view(shape_a)
    b = (torch.randn(*shape_b, generator=g).view(*shape_b[:-1], K // 32, 32) * blk(shape_b)).view(shape_b)
    pa = pack_mx(a.to(dev), "fp4_e2m1", nibbles=True)
    pb = pack_mx(b.to(dev), "fp4_e2m1", nibbles=True)
    got = gemm_nt(pa, pb, torch.float32)
    qa = unpack_mx(*pa, torch.float32).double()
    qb = unpack_mx(*pb, torch.float32).double()
    want = qa @ qb.transpose(-1, -2)
    assert got.shape == want.shape
    assert rel_err(got, want) < 1e-3
    den = qa.abs() @ qb.abs().transpose(-1, -2)
    assert ((got.double() - want).abs() <= 2e-4 * den + 1e-30).all()
    on_bytes = gemm_nt(pack_mx(a.to(dev), "fp4_e2m1"), pack_mx(b.to(dev), "fp4_e2m1"), torch.float32)
    assert rel_err(got, on_bytes) < 1e-3
    # 16-bit output with bias and epilogue quantization: the fp32 result pushed through the same steps
    from microxcaling_amd.elemwise_ops import _quantize_bfloat
    bias = torch.randn(N, generator=g).to(dev).to(torch.bfloat16)
    want16 = _quantize_bfloat(_quantize_bfloat(got.to(torch.bfloat16), 16, round="nearest") + bias, 16, round="nearest")
    got16 = gemm_nt(pa, pb, torch.bfloat16, bias=bias, epilogue_quant=True)
    assert torch.equal(got16.view(torch.int16), want16.view(torch.int16))
    with pytest.raises(RuntimeError, match="both operands"):
        gemm_nt(pa, pack_mx(b.to(dev), "fp4_e2m1"), torch.float32)


@pytest.mark.parametrize("fmt,K", [("fp8_e4m3", 128), ("fp4_e2m1", 256)])
@pytest.mark.parametrize("M,N,batch", [(2048, 2048, 16), (2000, 1990, 17), (130, 4100, 130)])
def test_one_step_products_with_thousands_of_tiles(dev, fmt, K, M, N, batch):
    """K of a single 128-byte step and thousands of output tiles (attention scores), full and ragged
    tiles: against the unpacked operands multiplied by torch, and bit for bit against the same product
    taken one batch entry at a time."""
    from microxcaling_amd.fused import pack_mx, gemm_nt, unpack_mx
    g = torch.Generator().manual_seed(M + N + batch)
    nib = fmt == "fp4_e2m1"
    a = torch.randn(batch, M, K, generator=g).to(torch.bfloat16).to(dev)
    b = torch.randn(batch, N, K, generator=g).to(torch.bfloat16).to(dev)
    pa, pb = pack_mx(a, fmt, nibbles=nib), pack_mx(b, fmt, nibbles=nib)
    got = gemm_nt(pa, pb, torch.float32)
    qa, qb = unpack_mx(*pa, torch.float32), unpack_mx(*pb, torch.float32)
    want = torch.bmm(qa.double(), qb.double().transpose(-1, -2))
    assert rel_err(got, want) < 1e-3
    den = torch.bmm(qa.abs(), qb.abs().transpose(-1, -2))
    assert ((got.double() - want).abs() <= 2e-4 * den + 1e-30).all()
    # bfloat16 quantization in the epilogue (plain-range form on whole pieces, general form where a
    # piece holds a zero or a NaN): the separate steps on the fp32 product, bit for bit
    from microxcaling_amd.elemwise_ops import _quantize_bfloat
    a2 = a.clone()
    a2[0, :40] = 0.0                                         # exact zeros in the product
    a2[1, 7, 3] = float("nan")
    pa2 = pack_mx(a2, fmt, nibbles=nib)
    want_q = _quantize_bfloat(gemm_nt(pa2, pb, torch.float32).to(torch.bfloat16), 16, round="nearest")
    got_q = gemm_nt(pa2, pb, torch.bfloat16, epilogue_quant=True)
    assert torch.equal(torch.isnan(got_q), torch.isnan(want_q))
    assert torch.equal(torch.nan_to_num(got_q).view(torch.int16), torch.nan_to_num(want_q).view(torch.int16))
    del want_q, got_q, a2, pa2
    bias = torch.randn(N, generator=g).to(dev).to(torch.bfloat16)
    got16 = gemm_nt(pa, pb, torch.bfloat16, bias=bias, epilogue_quant=True)
    for i in (0, batch // 2, batch - 1):
        one_a = tuple(t[i].contiguous() if torch.is_tensor(t) else t for t in pa)
        one_b = tuple(t[i].contiguous() if torch.is_tensor(t) else t for t in pb)
        assert torch.equal(gemm_nt(one_a, one_b, torch.float32), got[i])
        assert torch.equal(gemm_nt(one_a, one_b, torch.bfloat16, bias=bias, epilogue_quant=True).view(torch.int16),
                           got16[i].view(torch.int16))


@pytest.mark.parametrize("fmt", ["fp8_e4m3", "fp6_e2m3", "fp4_e2m1"])
def test_pack_with_the_bfloat16_quantizer_first(dev, fmt):
    """pack_mx(pre_bfloat16=True) = the elementwise bfloat16 / round-half-away quantizer, then pack_mx:
    bit for bit, on plain data and on rows with zeros, subnormals, Inf, NaN and the largest values."""
    from microxcaling_amd.elemwise_ops import _quantize_bfloat
    from microxcaling_amd.fused import pack_mx
    g = torch.Generator().manual_seed(31)
    x = (torch.randn(300, 256, generator=g) * torch.exp2(torch.randint(-8, 8, (300, 256), generator=g).float())).to(torch.bfloat16)
    x[3, :9] = torch.tensor([0.0, -0.0, float("inf"), float("-inf"), float("nan"), 1e-39, -1e-40, 3.38e38, -3.3e38]).to(torch.bfloat16)
    x[7] = 0.0
    x[9, 40:80] *= 1e-38
    xd = x.to(dev)
    two_steps = pack_mx(_quantize_bfloat(xd, 16, round="nearest"), fmt)
    one_step = pack_mx(xd, fmt, pre_bfloat16=True)
    assert torch.equal(one_step[0], two_steps[0]) and torch.equal(one_step[1], two_steps[1])
    with pytest.raises(RuntimeError, match="bf16"):
        pack_mx(xd.float(), fmt, pre_bfloat16=True)


@pytest.mark.parametrize("fn", ["bmm", "matmul"])
def test_inference_skips_the_operand_quantization_pass(dev, fn):
    """Without gradients mx.bmm / mx.matmul leave the bfloat16 quantization of their operands to the
    pack kernels: same output, bit for bit, as with gradients wanted (separate passes)."""
    from microxcaling_amd.bmm import bmm
    from microxcaling_amd.matmul import matmul
    specs = _specs(a_elem_format="fp6_e2m3", w_elem_format="fp6_e2m3", block_size=32, bfloat=16)
    g = torch.Generator().manual_seed(3)
    a = torch.randn(6, 200, 128, generator=g).to(torch.bfloat16).to(dev)
    b = torch.randn(6, 264, 128, generator=g).to(torch.bfloat16).to(dev).transpose(-1, -2)
    a[0, 0, :5] = 0.0
    f = bmm if fn == "bmm" else matmul
    plain = f(a, b, mx_specs=specs)
    with_grad = f(a.clone().requires_grad_(True), b, mx_specs=specs)
    assert with_grad.requires_grad and not plain.requires_grad
    assert torch.equal(plain.view(torch.int16), with_grad.detach().view(torch.int16))


@pytest.mark.parametrize("with_bias", [False, True])
@pytest.mark.parametrize("shape", [(640, 512, 768), (1030, 520, 1152), (70, 136, 256)])
def test_linear_inference_skips_the_operand_quantization_passes(dev, with_bias, shape):
    """mx.Linear under bfloat=16 without gradients: operands quantized by the pack kernels, product
    and bias sum by the GEMM's epilogue (plain-range form where it applies) -- bit for bit the output
    of the same layer with gradients wanted (separate passes), large and small tiles."""
    from microxcaling_amd.linear import Linear, linear
    M, N, K = shape
    specs = _specs(w_elem_format="fp8_e4m3", a_elem_format="fp8_e4m3", block_size=32, bfloat=16)
    g = torch.Generator().manual_seed(M + N)
    x = torch.randn(M, K, generator=g).to(torch.bfloat16).to(dev)
    x[0, :40] = 0.0
    w = (torch.randn(N, K, generator=g) * 0.05).to(torch.bfloat16).to(dev)
    w[3] = 0.0                                               # a column of exact zeros in the product
    b = torch.randn(N, generator=g).to(torch.bfloat16).to(dev) if with_bias else None
    plain = linear(x, w, b, mx_specs=specs)
    with_grad = linear(x.clone().requires_grad_(True), w, b, mx_specs=specs)
    assert with_grad.requires_grad and not plain.requires_grad
    assert torch.equal(plain.view(torch.int16), with_grad.detach().view(torch.int16))
    mod = Linear(K, N, bias=with_bias, mx_specs=specs).to(torch.bfloat16).to(dev)
    with torch.no_grad():
        mod.weight.copy_(w)
        if with_bias:
            mod.bias.copy_(b)
    assert torch.equal(mod(x).detach().view(torch.int16), plain.view(torch.int16))      # parameters want gradients
    with torch.no_grad():
        assert torch.equal(mod(x).view(torch.int16), plain.view(torch.int16))


@pytest.mark.parametrize("fmt", ["fp8_e4m3", "fp6_e2m3", "fp4_e2m1"])
@pytest.mark.parametrize("keep_dense", [True, False])
def test_prequantized_linear_keeps_the_packed_weight(dev, fmt, keep_dense):
    """Linear.prequantize_weights (mx/linear.py:246-274) on the fused path: the weight's MX codes and
    scales are built at the first forward pass and reused; outputs are bit for bit those of the same
    layer packing its bf16 weight on every call; keep_dense=False leaves only codes + scales."""
    from microxcaling_amd.linear import Linear, linear
    M, N, K = 640, 768, 512
    specs = _specs(w_elem_format=fmt, a_elem_format=fmt, block_size=32, bfloat=16, round="even")
    torch.manual_seed(11)
    lin = Linear(K, N, mx_specs=specs).to(dev).eval()
    g = torch.Generator().manual_seed(12)
    x = torch.randn(3, M, K, generator=g).to(torch.bfloat16).to(dev)
    lin.prequantize_weights(keep_dense=keep_dense)
    assert lin.weight.dtype == torch.bfloat16 and lin.packed_weight_bytes() == 0
    w, b = lin.weight.data.clone(), lin.bias.data.clone()
    with torch.no_grad():
        want = linear(x, w, b, mx_specs=specs, prequantized_weights=True)     # packs w on every call
        got1 = lin(x)
        got2 = lin(x[:, :100])                                                # reuses the codes
    assert torch.equal(got1.view(torch.int16), want.view(torch.int16))
    assert torch.equal(got2.view(torch.int16), want[:, :100].contiguous().view(torch.int16))
    per_weight = 0.5 if fmt == "fp4_e2m1" else 1.0
    assert lin.packed_weight_bytes() == int(N * K * per_weight) + N * K // 32
    assert lin.weight.numel() == (N * K if keep_dense else 0)
    # against the oracle (round-half-even everywhere), the tolerance of bf16 tensors
    ref = O.mx_linear_forward(x.cpu(), w.cpu(), b.cpu(), fmt, fmt, bfloat=16, round="even").float()
    diff = (got1.float().cpu() - ref).abs()
    assert bool((diff <= 2 ** -6 * (ref.abs() + b.float().cpu().abs()) + 2e-3 * ref.pow(2).mean().sqrt()).all())
    if keep_dense:
        # a changed weight is packed again
        with torch.no_grad():
            lin.weight.mul_(2.0)
            again = lin(x)
            assert torch.equal(again.view(torch.int16),
                               linear(x, lin.weight.data, b, mx_specs=specs, prequantized_weights=True).view(torch.int16))
        assert not torch.equal(again, got1)


def test_gemm_propagates_nan_blocks(dev):
    from microxcaling_amd.fused import pack_mx, gemm_nt
    a = torch.randn(128, 128)
    a[5, 40] = float("inf")
    b = torch.randn(128, 128)
    out = gemm_nt(pack_mx(a.to(dev), "fp8_e4m3"), pack_mx(b.to(dev), "fp8_e4m3")).cpu()
    assert torch.isnan(out[5]).all() and torch.isfinite(out[torch.arange(128) != 5]).all()


def _specs(**kw):
    from microxcaling_amd.specs import finalize_mx_specs
    return finalize_mx_specs(dict(kw))


@pytest.mark.parametrize("fused", [False, True])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_linear_forward_matches_reference_forward(dev, fused, dtype):
    """mx.Linear forward (the benchmark's MXFP8 linear layer at a reduced size): quantize-then-fp32-matmul oracle,
    relative tolerance 1e-3 (max |diff| / RMS of the output)."""
    from microxcaling_amd import gemm
    from microxcaling_amd.linear import linear
    g = torch.Generator().manual_seed(4)
    x = torch.randn(512, 1024, generator=g).to(dtype)
    w = (torch.randn(384, 1024, generator=g) * 0.02).to(dtype)
    b = torch.randn(384, generator=g).to(dtype)
    specs = _specs(w_elem_format="fp8_e4m3", a_elem_format="fp8_e4m3", block_size=32)
    want = O.mx_linear_forward(x, w, b, "fp8_e4m3", "fp8_e4m3")      # same dtype as the GPU run
    gemm.set_fused(fused)
    try:
        got = linear(x.to(dev), w.to(dev), b.to(dev), mx_specs=specs)
    finally:
        gemm.set_fused(True)
    torch.cuda.synchronize()
    assert got.dtype == dtype
    if dtype == torch.float32:
        assert rel_err(got, want) < 1e-3
    else:
        # bf16 tensors round the product and then the bias sum to bf16: allow one bf16 ulp of the
        # larger of the two (|product| <= |result| + |bias|) on top of the accumulation tolerance
        diff = (got.float().cpu() - want.float()).abs()
        rms = want.float().pow(2).mean().sqrt()
        mag = want.float().abs() + b.float().abs().view(1, -1)
        assert (diff <= 2 ** -6 * mag + 2e-3 * rms).all()


@pytest.mark.parametrize("fused", [False, True])
def test_bmm_and_softmax_forward(dev, fused):
    """mx.bmm Q.K^T with MXFP6 e2m3 along head_dim, then the bfloat16 softmax chain (config 5 at a
    reduced size).  Logits: relative 1e-3; softmax: absolute 2^-8 (one bf16 ulp at 1.0)."""
    from microxcaling_amd import gemm
    from microxcaling_amd.bmm import bmm
    from microxcaling_amd.softmax import softmax
    g = torch.Generator().manual_seed(5)
    q = torch.randn(4, 256, 128, generator=g)
    k = torch.randn(4, 256, 128, generator=g)
    specs = _specs(a_elem_format="fp6_e2m3", block_size=32, bfloat=16)
    want = O.mx_bmm_forward(q, k.transpose(-1, -2), "fp6_e2m3", bfloat=16)
    gemm.set_fused(fused)
    try:
        got = bmm(q.to(dev), k.to(dev).transpose(-1, -2), mx_specs=specs)
    finally:
        gemm.set_fused(True)
    torch.cuda.synchronize()
    assert rel_err(got, want) < 1e-2                      # logits are re-rounded to bfloat16
    sm = softmax(got, dim=-1, mx_specs=specs).cpu()
    sm_want = O.softmax_forward(want, -1, bfloat=16)
    assert (sm - sm_want).abs().max() <= 2 ** -8 * 4


def _grid_step_apart(got, want, share=0.02):
    """Probabilities after the bfloat16 quantizer with round-half-away lie on a grid of even bf16
    significands: neighbours are 2^-6 of their value apart at most (2^-7 just below 1.0).  One such
    step (two on at most one element in 10 000), and at most `share` of the elements different at all
    (far below 2^-126 the step is that of bf16's subnormals)."""
    d = (got - want).abs()
    steps = d / (2 ** -6 * want.abs() + 2.0 ** -133)
    assert steps.max().item() <= 2.0, steps.max().item()            # a step in the row sum and one in the value
    assert (steps > 1.0).float().mean().item() <= 1e-4, (steps > 1.0).float().mean().item()
    assert (d > 0).float().mean().item() <= share, (d > 0).float().mean().item()


@pytest.mark.parametrize("shape", [(4, 256, 2048), (1, 70, 64), (3, 33, 544), (2, 2048, 1024), (130, 32, 32)])
@pytest.mark.parametrize("fmt,exp2", [("fp6_e2m3", False), ("fp8_e4m3", True), ("fp8_e5m2", False), ("fp4_e2m1", False)])
def test_bmm_softmax_in_one_launch(dev, shape, fmt, exp2):
    """mx.bmm_softmax (attention scores, logits kept in registers) against (1) mx.softmax(mx.bmm(...)),
    the two separate kernels, and (2) the oracle's softmax chain on the logits those kernels produced:
    absolute 2^-8 (one bf16 step at 1.0), at most 2 % of the elements different at all -- the
    tolerance the separate softmax kernel has against the CPU chain (exp, order of the row sum)."""
    from microxcaling_amd.bmm import bmm, bmm_softmax
    from microxcaling_amd.softmax import softmax
    B, M, N = shape
    specs = _specs(a_elem_format=fmt, block_size=32, bfloat=16, softmax_exp2=exp2)
    g = torch.Generator().manual_seed(B * 7 + M + N)
    q = torch.randn(B, M, 128, generator=g).to(torch.bfloat16).to(dev)
    k = (torch.randn(B, N, 128, generator=g) * (0.3 if fmt == "fp8_e5m2" else 1.0)).to(torch.bfloat16).to(dev)
    q[0, 0] = 0.0                                            # a row of zero logits: uniform probabilities
    k[0, 5, :32] = 0.0
    got = bmm_softmax(q, k.transpose(-1, -2), mx_specs=specs)
    logits = bmm(q, k.transpose(-1, -2), mx_specs=specs)
    two = softmax(logits, dim=-1, mx_specs=specs)
    torch.cuda.synchronize()
    assert got.shape == two.shape and got.dtype == torch.bfloat16
    _grid_step_apart(got.float(), two.float())
    want = O.softmax_forward(logits.cpu(), -1, bfloat=16, use_exp2=exp2).float()
    _grid_step_apart(got.float().cpu(), want)
    assert torch.equal(got[0, 0].float().cpu(), want[0, 0])  # zero logits: exp(0) = 1 exactly, sum = N exactly


def test_bmm_softmax_special_values_and_general_form(dev):
    """Workgroups that leave the plain range (an Inf / NaN block, huge or tiny logits) take the
    element-by-element form: NaN rows where the chain gives NaN rows, same tolerance elsewhere; and
    that form, forced for every workgroup, agrees with the packed one on ordinary data."""
    from microxcaling_amd import custom_extensions as ce
    from microxcaling_amd.bmm import bmm, bmm_softmax
    from microxcaling_amd.softmax import softmax
    specs = _specs(a_elem_format="fp8_e4m3", block_size=32, bfloat=16)
    g = torch.Generator().manual_seed(21)
    q = torch.randn(3, 96, 128, generator=g).to(torch.bfloat16)
    k = torch.randn(3, 160, 128, generator=g).to(torch.bfloat16)
    q[0, 3, 7] = float("inf")                                # NaN block -> row 3 of batch 0 is NaN
    k[1, 9, 100] = float("nan")                              # -> column 9 of batch 1 is NaN -> every row NaN
    q[2, :32] *= 2.0 ** 60                                   # logits around 2^120: outside the plain range
    k[2, :80] *= 2.0 ** 60
    q[2, 64:] *= 2.0 ** -70                                  # and around 2^-140 ... 2^-10
    qd, kd = q.to(dev), k.to(dev)
    got = bmm_softmax(qd, kd.transpose(-1, -2), mx_specs=specs)
    two = softmax(bmm(qd, kd.transpose(-1, -2), mx_specs=specs), dim=-1, mx_specs=specs)
    torch.cuda.synchronize()
    assert torch.equal(torch.isnan(got), torch.isnan(two))
    assert bool(torch.isnan(got[0, 3]).all()) and bool(torch.isnan(got[1]).all()) and not bool(torch.isnan(got[0, 4]).any())
    fin = ~torch.isnan(two)
    _grid_step_apart(got.float()[fin], two.float()[fin])
    q2 = torch.randn(2, 64, 128, generator=g).to(torch.bfloat16).to(dev)
    k2 = torch.randn(2, 2048, 128, generator=g).to(torch.bfloat16).to(dev)
    packed = bmm_softmax(q2, k2.transpose(-1, -2), mx_specs=specs)
    ce.set_general_form(True)
    try:
        general = bmm_softmax(q2, k2.transpose(-1, -2), mx_specs=specs)
    finally:
        ce.set_general_form(False)
    _grid_step_apart(packed.float(), general.float(), share=0.01)


def test_bmm_softmax_declines_what_it_does_not_cover(dev):
    """Other head dims, row lengths, gradients, fp32 tensors: the two separate ops run, same values
    as calling them directly."""
    from microxcaling_amd.bmm import bmm, bmm_softmax
    from microxcaling_amd.softmax import softmax
    specs = _specs(a_elem_format="fp6_e2m3", block_size=32, bfloat=16)
    g = torch.Generator().manual_seed(22)
    for shape_q, shape_k, dt in (((2, 40, 64), (2, 96, 64), torch.bfloat16), ((2, 40, 128), (2, 100, 128), torch.bfloat16),
                                 ((2, 40, 128), (2, 96, 128), torch.float32)):
        q = torch.randn(*shape_q, generator=g).to(dt).to(dev)
        k = torch.randn(*shape_k, generator=g).to(dt).to(dev)
        a = bmm_softmax(q, k.transpose(-1, -2), mx_specs=specs)
        b = softmax(bmm(q, k.transpose(-1, -2), mx_specs=specs), dim=-1, mx_specs=specs)
        assert torch.equal(a, b)
    q = torch.randn(2, 40, 128, generator=g).to(torch.bfloat16).to(dev).requires_grad_(True)
    k = torch.randn(2, 96, 128, generator=g).to(torch.bfloat16).to(dev)
    out = bmm_softmax(q, k.transpose(-1, -2), mx_specs=specs)
    out.sum().backward()
    assert q.grad is not None and torch.isfinite(q.grad).all()


def test_linear_backward_runs(dev):
    from microxcaling_amd.linear import Linear
    specs = _specs(w_elem_format="fp6_e3m2", a_elem_format="fp6_e3m2", block_size=32, bfloat=16)
    lin = Linear(256, 128, mx_specs=specs).to(dev)
    x = torch.randn(64, 256, device=dev, requires_grad=True)
    lin(x).sum().backward()
    assert x.grad.shape == x.shape and lin.weight.grad.shape == lin.weight.shape
    assert torch.isfinite(x.grad).all()


# ---- fused softmax kernel against the oracle's chain of tensor ops --------------------------------
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("shape", [(3, 5, 2048), (64, 1000), (7, 8), (2, 4096), (33, 264),
                                   # two and four waves per row; row counts that leave waves of a block spare
                                   (5, 8192), (3, 6000), (5, 16384), (2, 3, 12000)])
@pytest.mark.parametrize("spec", [dict(bfloat=16), dict(bfloat=16, softmax_exp2=True),
                                  dict(bfloat=16, vec_use_exp2=True, vec_use_recip=True),
                                  dict(bfloat=16, round="floor"), dict(bfloat=16, round="even"),
                                  dict(fp=16), dict(bfloat=12), dict(fp=10, round="even"),
                                  dict(fp=16, round="even"), dict()])
def test_fused_softmax_against_chain(dev, dtype, shape, spec):
    """One-kernel softmax vs the reference's chain (max, sub, exp, sum, div, each followed by the
    elementwise quantizer) on the CPU.  exp and the order of the row sum differ in the last bit
    between the two, which the quantizer can turn into one step of the element format: tolerance
    2^-8 absolute (one bf16 step at 1.0) and 1 % of the elements allowed to differ at all
    (floor rounding: 3 %)."""
    from microxcaling_amd.softmax import softmax, _fused_forward
    from microxcaling_amd.specs import apply_mx_specs
    g = torch.Generator().manual_seed(sum(shape))
    x = (torch.randn(*shape, generator=g) * 3).to(dtype)
    x[0, ..., 3] = 9.5                                   # a clear maximum somewhere
    specs = _specs(**spec)
    if specs is not None:                                # the kernel is the path under test
        bits = spec["bfloat"] - 7 if "bfloat" in spec else spec.get("fp", 11) - 4
        unfusable = dtype == torch.bfloat16 and spec.get("round") == "even" and bits >= 9 \
            and spec.get("bfloat") != 16
        assert (_fused_forward(x.to(dev), x.dim() - 1, apply_mx_specs(specs)) is None) == unfusable
    got = softmax(x.to(dev), dim=-1, mx_specs=specs).cpu()
    want = O.softmax_forward(x, -1, bfloat=spec.get("bfloat", 0), fp=spec.get("fp", 0),
                             round=spec.get("round", "nearest"), use_exp2=spec.get("softmax_exp2", False),
                             vec_use_exp2=spec.get("vec_use_exp2", False),
                             vec_use_recip=spec.get("vec_use_recip", False))
    assert got.dtype == want.dtype and got.shape == want.shape
    diff = (got.float() - want.float()).abs()
    assert diff.max().item() <= 2.0 ** -8
    if specs is None:                                    # the reference then calls torch's softmax
        plain = torch.softmax(x, -1).float()
        assert torch.allclose(got.float(), plain, rtol=2.0 ** -7 if dtype == torch.bfloat16 else 1e-5, atol=1e-9)
        return
    frac = (diff > 0).float().mean().item()
    assert frac <= (0.03 if spec.get("round") == "floor" else 0.01), frac


def test_fused_softmax_special_rows(dev):
    """Rows holding -inf, +inf and NaN: -inf entries get weight 0; a row with +inf or NaN is NaN
    throughout (inf - inf), exactly like the chain of tensor ops."""
    from microxcaling_amd.softmax import softmax
    x = torch.randn(6, 64)
    x[1, 5] = float("-inf")
    x[2, 7] = float("inf")
    x[3, 9] = float("nan")
    x[4, :] = float("-inf")
    specs = _specs(bfloat=16)
    got = softmax(x.to(dev), dim=-1, mx_specs=specs).cpu()
    want = O.softmax_forward(x, -1, bfloat=16)
    assert torch.equal(torch.isnan(got), torch.isnan(want))
    assert got[1, 5] == 0 and torch.isnan(got[2]).all() and torch.isnan(got[3]).all() and torch.isnan(got[4]).all()
    ok = ~torch.isnan(want)
    assert (got[ok] - want[ok]).abs().max() <= 2.0 ** -8


@pytest.mark.parametrize("shape", [(64, 2048), (9, 264), (6, 8192), (5, 16384)])
@pytest.mark.parametrize("spec", [dict(bfloat=16), dict(bfloat=16, softmax_exp2=True),
                                  dict(bfloat=16, vec_use_exp2=True, vec_use_recip=True)])
def test_fused_softmax_plain_and_general_forms_agree(dev, shape, spec):
    """bf16 rows whose values all lie in [2^-100, 2^100) are quantized without the special cases of
    the closed form; any other row takes the general form.  A row with one entry at -200 and the
    same row with -inf there must come out bit-identical: both entries weigh exactly 0, and only
    the second row holds a special value."""
    from microxcaling_amd.softmax import softmax
    g = torch.Generator().manual_seed(shape[1])
    x = (torch.randn(*shape, generator=g) * 3).to(torch.bfloat16)
    x[x == 0] = 1.0
    y = x.clone()
    cols = torch.arange(shape[0]) * 37 % shape[1]
    x[torch.arange(shape[0]), cols] = -200.0
    y[torch.arange(shape[0]), cols] = float("-inf")
    specs = _specs(**spec)
    got_plain = softmax(x.to(dev), dim=-1, mx_specs=specs).cpu()
    got_general = softmax(y.to(dev), dim=-1, mx_specs=specs).cpu()
    assert (got_plain[torch.arange(shape[0]), cols] == 0).all()
    assert torch.equal(got_plain.view(torch.int16), got_general.view(torch.int16))


def test_fused_softmax_bf16_rows_outside_the_plain_range(dev):
    """Huge, tiny, zero and subnormal bf16 logits against the chain of tensor ops."""
    from microxcaling_amd.softmax import softmax
    g = torch.Generator().manual_seed(5)
    x = torch.randn(8, 256, generator=g).to(torch.bfloat16)
    x[0, 3] = 2.0 ** 101                                 # maximum beyond the plain range
    x[1] = x[1] * 2.0 ** -110                            # every entry below it
    x[2, 10:20] = 0.0
    x[3, 7] = -0.0
    x[4, 5] = 2.0 ** -130                                # bf16 subnormal
    x[5, ::2] = 2.0 ** 100
    x[6] = x[6] * 2.0 ** 99
    specs = _specs(bfloat=16)
    got = softmax(x.to(dev), dim=-1, mx_specs=specs).cpu()
    want = O.softmax_forward(x, -1, bfloat=16)
    assert torch.equal(torch.isnan(got), torch.isnan(want))
    ok = ~torch.isnan(want)
    assert (got[ok].float() - want[ok].float()).abs().max() <= 2.0 ** -8
    assert got[0, 3] == 1 and got[0].float().sum() == 1


def test_softmax_unfused_path_still_matches(dev):
    from microxcaling_amd import gemm
    from microxcaling_amd.softmax import softmax
    x = torch.randn(16, 2048).to(torch.bfloat16)
    specs = _specs(bfloat=16)
    gemm.set_fused(False)
    try:
        a = softmax(x.to(dev), dim=-1, mx_specs=specs).cpu()
    finally:
        gemm.set_fused(True)
    b = softmax(x.to(dev), dim=-1, mx_specs=specs).cpu()
    assert (a.float() - b.float()).abs().max() <= 2.0 ** -8
    # another axis than the last one is served by the separate steps
    c = softmax(x.to(dev), dim=0, mx_specs=specs).cpu()
    assert (c.float() - O.softmax_forward(x, 0, bfloat=16).float()).abs().max() <= 2.0 ** -8


# ---- backward passes against the oracle's restatement --------------------------------------------
def _close(got, want, rel, coarse=False):
    """coarse: the result passed a bfloat16 quantizer, which turns a last-bit difference of the GEMM
    into one bfloat16 step now and then: one step of the largest entry, on at most 2 % of them."""
    got, want = got.float().cpu(), want.float()
    assert got.shape == want.shape
    rms = want.pow(2).mean().sqrt().item() + 1e-30
    diff = (got - want).abs()
    if coarse:
        assert diff.max().item() <= 2.0 ** -6 * want.abs().max().item(), (diff.max().item(), want.abs().max().item())
        assert (diff > rel * rms).float().mean().item() <= 0.02
    else:
        assert diff.max().item() <= rel * rms, (diff.max().item(), rms)


@pytest.mark.parametrize("dtype,rel", [(torch.float32, 1e-3), (torch.bfloat16, 4e-2)])
@pytest.mark.parametrize("bfloat", [0, 16])
def test_linear_backward_against_oracle(dev, dtype, rel, bfloat):
    """grad_input / grad_weight / grad_bias of mx.Linear (MXFP8 e4m3 forward and backward) vs the
    oracle's restatement of mx/linear.py:103-198 on the CPU.  The operands of every contraction are
    bit-identical on both sides; fp32: only the summation order differs (1e-3 of the RMS);
    bf16: the GEMM output is rounded to bf16, so one bf16 step of the largest entries (4e-2 RMS)."""
    from microxcaling_amd.linear import linear
    g = torch.Generator().manual_seed(21)
    x = torch.randn(4, 64, 128, generator=g).to(dtype)            # 256 examples: the gradient GEMMs
    w = (torch.randn(128, 128, generator=g) * 0.1).to(dtype)      # qualify for the packed path too
    b = torch.randn(128, generator=g).to(dtype)
    go = torch.randn(4, 64, 128, generator=g).to(dtype)
    specs = _specs(w_elem_format="fp8_e4m3", a_elem_format="fp8_e4m3", block_size=32, bfloat=bfloat,
                   quantize_backprop=True)
    xd, wd, bd = (t.to(dev).requires_grad_(True) for t in (x, w, b))
    out = linear(xd, wd, bd, mx_specs=specs)
    out.backward(go.to(dev))
    gi, gw, gb = O.mx_linear_backward(x, w, go, True, "fp8_e4m3", bfloat=bfloat)
    coarse = bfloat == 16 or dtype == torch.bfloat16
    _close(xd.grad, gi, rel, coarse)
    _close(wd.grad, gw, rel, coarse)
    _close(bd.grad, gb, rel, coarse)


@pytest.mark.parametrize("dtype,rel", [(torch.float32, 1e-3), (torch.bfloat16, 4e-2)])
def test_bmm_backward_against_oracle(dev, dtype, rel):
    from microxcaling_amd.bmm import bmm
    g = torch.Generator().manual_seed(22)
    a = torch.randn(4, 128, 128, generator=g).to(dtype)
    b = torch.randn(4, 128, 256, generator=g).to(dtype)
    go = torch.randn(4, 128, 256, generator=g).to(dtype)
    specs = _specs(a_elem_format="fp6_e2m3", block_size=32, quantize_backprop=True)
    ad, bd = a.to(dev).requires_grad_(True), b.to(dev).requires_grad_(True)
    bmm(ad, bd, mx_specs=specs).backward(go.to(dev))
    g1, g2 = O.mx_bmm_backward(a, b, go, "fp6_e2m3")
    _close(ad.grad, g1, rel, dtype == torch.bfloat16)
    _close(bd.grad, g2, rel, dtype == torch.bfloat16)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("exp2", [False, True])
def test_softmax_backward_against_oracle(dev, dtype, exp2):
    """Backward of the bfloat16 softmax from the same saved output on both sides: only the order of
    the row sum differs."""
    from microxcaling_amd.softmax import softmax
    g = torch.Generator().manual_seed(23)
    x = (torch.randn(8, 256, generator=g) * 2).to(dtype)
    go = torch.randn(8, 256, generator=g).to(dtype)
    specs = _specs(bfloat=16, softmax_exp2=exp2, quantize_backprop=True)
    xd = x.to(dev).requires_grad_(True)
    out = softmax(xd, dim=-1, mx_specs=specs)
    out.backward(go.to(dev))
    want = O.softmax_backward(out.detach().cpu(), go, -1, bfloat=16, use_exp2=exp2)
    diff = (xd.grad.float().cpu() - want.float()).abs()
    assert diff.max().item() <= 2.0 ** -7 * want.float().abs().max().item()
    assert (diff > 0).float().mean().item() < 0.02


_ACTS = {
    "sigmoid": lambda A, x, s: A.sigmoid(x, mx_specs=s),
    "tanh": lambda A, x, s: A.tanh(x, mx_specs=s),
    "silu": lambda A, x, s: A.silu(x, mx_specs=s),
    "gelu": lambda A, x, s: A.gelu(x, mx_specs=s),
    "gelu_first_order": lambda A, x, s: A.gelu(x, mx_specs=s, first_order_gelu=True),
}


def _one_step_apart(got, want, frac_allowed):
    """exp / tanh differ in the last bit between the GPU and the CPU library; a quantizer turns that
    into one step of the format now and then.  At most two steps of the coarsest grid in play
    (2^-6 relative), on at most `frac_allowed` of the elements; NaNs in the same places."""
    got, want = got.float().cpu(), want.float().cpu()
    assert got.shape == want.shape
    assert torch.equal(torch.isnan(got), torch.isnan(want))
    ok = ~torch.isnan(want)
    g, w = got[ok], want[ok]
    inf = torch.isinf(w)
    assert torch.equal(g[inf], w[inf])
    d = (g[~inf] - w[~inf]).abs()
    assert (d <= 2.0 ** -5 * w[~inf].abs() + 1e-37).all(), d.max().item()
    assert (d > 0).float().mean().item() <= frac_allowed


@pytest.mark.parametrize("act", sorted(_ACTS))
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("spec", [dict(bfloat=16), dict(bfloat=16, vec_use_exp2=True), dict(bfloat=12),
                                  dict(bfloat=16, round="floor")],
                         ids=["bfloat16", "bfloat16-exp2", "bfloat12", "bfloat16-floor"])
def test_fused_activation_against_chain(dev, act, dtype, spec):
    """One-kernel activation forward (and the backward pass fed by what it saved) against the chain
    of vec_* ops on the CPU, which is bit-identical to the reference's layers."""
    from microxcaling_amd import activations as A, gemm
    from microxcaling_amd.specs import apply_mx_specs
    specs = _specs(**spec)
    g = torch.Generator().manual_seed(len(act) + spec.get("bfloat", 0))
    x = (torch.randn(257, 130, generator=g) * 3).to(dtype)            # 33410 elements: a ragged tail
    w = torch.randn(257, 130, generator=g).to(dtype)
    outs = {}
    for where in ("cpu", "gpu"):
        xi = (x.to(dev) if where == "gpu" else x.clone()).requires_grad_(True)
        y = _ACTS[act](A, xi, specs)
        (y * (w.to(dev) if where == "gpu" else w)).sum().backward()
        outs[where] = (y.detach(), xi.grad.detach())
    assert A._fused_forward(x.to(dev), A.ACT_TANH, apply_mx_specs(specs)) is not None      # the path under test
    assert outs["gpu"][0].dtype == outs["cpu"][0].dtype
    loose = 0.06 if spec.get("round") == "floor" else 0.03
    _one_step_apart(outs["gpu"][0], outs["cpu"][0], loose)
    _one_step_apart(outs["gpu"][1], outs["cpu"][1], 2 * loose)
    # the separate steps on the GPU give the same as the kernel, to the same tolerance
    gemm.set_fused(False)
    try:
        y_chain = _ACTS[act](A, x.to(dev), specs)
    finally:
        gemm.set_fused(True)
    _one_step_apart(outs["gpu"][0], y_chain, loose)


@pytest.mark.parametrize("act", sorted(_ACTS))
@pytest.mark.parametrize("spec", [dict(bfloat=16), dict(bfloat=16, vec_use_exp2=True)], ids=["exp", "exp2"])
def test_fused_activation_plain_and_general_forms_agree(dev, act, spec):
    """bf16 inputs with 2^-20 <= |x| < 8 are quantized without the special cases of the closed form,
    wave by wave; one value outside that range sends its wave through the general form.  The
    results of all other elements must not depend on which form their wave took."""
    from microxcaling_amd import activations as A
    specs = _specs(**spec)
    g = torch.Generator().manual_seed(len(act))
    n = 512 * 300
    x = (torch.randn(n, generator=g) * 2.5).clamp(-7.9, 7.9)
    x[x.abs() < 2.0 ** -19] = 0.5
    x[:4096] = torch.exp2(torch.linspace(-19.9, 2.99, 4096)) * (1 - 2 * (torch.arange(4096) % 2))   # the whole range
    x = x.to(torch.bfloat16)
    assert ((x.float().abs() >= 2.0 ** -20) & (x.float().abs() < 8)).all()
    y = x.clone()
    hit = torch.arange(300) * 512 + torch.arange(300) * 7 % 512      # one per wave and iteration
    y[hit] = torch.tensor([0.0, float("inf"), 100.0, 2.0 ** -30, -8.0, float("nan")]).to(torch.bfloat16).repeat(50)
    got_plain = _ACTS[act](A, x.to(dev), specs).cpu()
    got_general = _ACTS[act](A, y.to(dev), specs).cpu()
    keep = torch.ones(n, dtype=torch.bool)
    keep[hit] = False
    assert torch.equal(got_plain[keep].view(torch.int16), got_general[keep].view(torch.int16))
    _one_step_apart(got_plain, _ACTS[act](A, x, specs), 0.03)


@pytest.mark.parametrize("act", sorted(_ACTS))
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_fused_activation_special_values(dev, act, dtype):
    from microxcaling_amd import activations as A
    specs = _specs(bfloat=16)
    x = torch.tensor([0.0, -0.0, float("inf"), float("-inf"), float("nan"), 1e-30, -1e-30, 88.0, -88.0,
                      100.0, -100.0, 3e38, -3e38, 1e-40, 20.0, -20.0], dtype=torch.float32).to(dtype)
    got = _ACTS[act](A, x.to(dev), specs)
    want = _ACTS[act](A, x, specs)
    _one_step_apart(got, want, 0.2)


@pytest.mark.parametrize("act", sorted(_ACTS))
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("spec", [dict(bfloat=16), dict(bfloat=12), dict(bfloat=16, round="floor"),
                                  dict(bfloat=16, quantize_backprop=False)],
                         ids=["bfloat16", "bfloat12", "bfloat16-floor", "no-backprop-quantization"])
def test_fused_activation_backward_equals_chain(dev, act, dtype, spec):
    """The backward kernel has only exact arithmetic and the quantizer in it: from the same saved
    tensors it must give the chain of vec_* ops bit for bit (special values included)."""
    from microxcaling_amd import activations as A, gemm
    specs = _specs(**spec)
    g = torch.Generator().manual_seed(len(act))
    x = (torch.randn(130, 257, generator=g) * 3).to(dtype)
    x[0, :8] = torch.tensor([0.0, -0.0, float("inf"), float("-inf"), float("nan"), 1e-30, 88.0, -88.0]).to(dtype)
    grad = (torch.randn(130, 257, generator=g) * torch.exp2(torch.randint(-20, 20, (130, 257), generator=g).float())).to(dtype)
    grad[1, :3] = torch.tensor([float("inf"), float("nan"), 0.0]).to(dtype)
    xi = x.to(dev).requires_grad_(True)
    y = _ACTS[act](A, xi, specs)
    grads = []
    for fused in (True, False):
        gemm.set_fused(fused)
        try:
            xi.grad = None
            y.backward(grad.to(dev), retain_graph=True)
            grads.append(xi.grad.clone())
        finally:
            gemm.set_fused(True)
    assert_bits_equal(grads[0].cpu(), grads[1].cpu(), act)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("spec", [dict(bfloat=16), dict(bfloat=16, softmax_exp2=True), dict(bfloat=12)],
                         ids=["bfloat16", "bfloat16-exp2", "bfloat12"])
@pytest.mark.parametrize("shape", [(3, 5, 2048), (64, 1000), (33, 264), (5, 8192), (3, 16384)])
def test_fused_softmax_backward_against_chain(dev, dtype, spec, shape):
    """One-kernel softmax backward against the chain of vec_* ops on the same saved output; only the
    order of the row sum differs."""
    from microxcaling_amd import gemm
    from microxcaling_amd.softmax import softmax
    specs = _specs(**spec)
    g = torch.Generator().manual_seed(sum(shape))
    x = (torch.randn(*shape, generator=g) * 3).to(dtype).to(dev).requires_grad_(True)
    grad = torch.randn(*shape, generator=g).to(dtype).to(dev)
    y = softmax(x, dim=-1, mx_specs=specs)
    grads = []
    for fused in (True, False):
        gemm.set_fused(fused)
        try:
            x.grad = None
            y.backward(grad, retain_graph=True)
            grads.append(x.grad.clone())
        finally:
            gemm.set_fused(True)
    got, want = grads[0].float().cpu(), grads[1].float().cpu()
    scale = want.abs().max().item()
    d = (got - want).abs()
    assert d.max().item() <= 2.0 ** -6 * scale
    assert (d > 0).float().mean().item() <= 0.05


@pytest.mark.parametrize("kind", ["layernorm", "rmsnorm"])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("spec", [dict(bfloat=16), dict(bfloat=12)], ids=["bfloat16", "bfloat12"])
@pytest.mark.parametrize("shape", [(6, 40, 1024), (257, 264), (9, 4096), (5, 8192), (3, 16384)])
def test_fused_norm_backward_against_chain(dev, kind, dtype, spec, shape):
    """One-kernel gradient with respect to the input of LayerNorm / RMSNorm against the chain of
    vec_* ops from the same saved tensors; only the order of the two row sums differs.  The
    parameter gradients come from the same separate steps either way."""
    from microxcaling_amd import gemm, layernorm as L
    specs = _specs(**spec)
    g = torch.Generator().manual_seed(sum(shape))
    n = shape[-1]
    mod = (L.LayerNorm if kind == "layernorm" else L.RMSNorm)(n, eps=1e-5, mx_specs=specs)
    with torch.no_grad():
        mod.weight.copy_(1 + 0.3 * torch.randn(n, generator=g))
        mod.bias.copy_(0.1 * torch.randn(n, generator=g))
    mod = mod.to(dtype).to(dev)
    x = (torch.randn(*shape, generator=g) * 2 + 0.5).to(dtype).to(dev).requires_grad_(True)
    grad = torch.randn(*shape, generator=g).to(dtype).to(dev)
    y = mod(x)
    res = []
    for fused in (True, False):
        gemm.set_fused(fused)
        try:
            x.grad = None
            mod.weight.grad = None
            y.backward(grad, retain_graph=True)
            res.append((x.grad.clone(), mod.weight.grad.clone()))
        finally:
            gemm.set_fused(True)
    step = 2.0 ** -7 if spec["bfloat"] == 16 else 2.0 ** -3        # one step of the format, relative
    gw, gw_want = res[0][1].float().cpu(), res[1][1].float().cpu()
    assert ((gw - gw_want).abs() <= step * gw_want.abs() + 1e-4 * gw_want.abs().max()).all()
    got, want = res[0][0].float().cpu(), res[1][0].float().cpu()
    d = (got - want).abs()
    assert d.max().item() <= 2.0 ** -5 * want.abs().max().item()
    assert (d > 0).float().mean().item() <= 0.08


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("spec", [dict(bfloat=16), dict(bfloat=12), dict(bfloat=14, round="floor")],
                         ids=["bfloat16", "bfloat12", "bfloat14-floor"])
@pytest.mark.parametrize("shape", [(1, 8), (5, 264), (257, 264), (6, 40, 1024), (4099, 520), (3, 16384),
                                   (2048, 4096), (70000, 64)])
def test_fused_norm_param_grads(dev, dtype, spec, shape):
    """Weight and bias gradients of LayerNorm / RMSNorm as column-sum kernels against (a) the separate
    steps (vec_mul, torch.sum, quantizer) on the GPU and (b) column sums in fp64 of the same quantized
    products, quantized on the CPU: the order of an fp32 sum is all that differs, so a result is the
    same number or, where the sum lies at a rounding boundary, the neighbouring one."""
    from microxcaling_amd import gemm, layernorm as L
    from microxcaling_amd.specs import apply_mx_specs
    from microxcaling_amd.vector_ops import vec_mul, vec_quantize
    specs = apply_mx_specs(_specs(**spec))
    gen = torch.Generator().manual_seed(sum(shape))
    g = vec_quantize((torch.randn(*shape, generator=gen) * 0.7 + 0.05).to(dtype).to(dev), mx_specs=specs)
    z = (torch.randn(*shape, generator=gen) * 1.5).to(dtype).to(dev)
    fused = L._fused_param_grads(g, z, specs)
    assert fused is not None
    # the packed plain-range form (bf16 tensors, bfloat16) and the general form add the same values in
    # the same order: bit for bit, also with zeros, tiny and huge values in some rows
    g2, z2 = g.clone(), z.clone()
    g2.view(-1, shape[-1])[0, :4] = 0.0
    z2.view(-1, shape[-1])[-1, :3] = torch.tensor([1e-30, 3e38, float("inf")]).to(dtype).to(dev)
    for gg, zz in ((g, z), (g2, z2)):
        a = L._fused_param_grads(gg, zz, specs)
        with _general_form():
            b = L._fused_param_grads(gg, zz, specs)
        assert torch.equal(torch.nan_to_num(a[0].float()), torch.nan_to_num(b[0].float()))
        assert torch.equal(torch.isnan(a[0]), torch.isnan(b[0])) and torch.equal(a[1], b[1])
    gemm.set_fused(False)
    try:
        assert L._fused_param_grads(g, z, specs) is None
        want_w, want_b = L._param_grads(g, z, specs)
        prod = vec_mul(g, z, mx_specs=specs)
    finally:
        gemm.set_fused(True)
    n = shape[-1]
    bits = spec["bfloat"]
    step = 2.0 ** -(bits - 9)                                 # one step of the format, relative
    for got, want, terms in ((fused[0], want_w, prod), (fused[1], want_b, g)):
        assert got.dtype == want.dtype and got.shape == want.shape == (n,)
        got, want = got.double().cpu(), want.double().cpu()
        terms = terms.double().reshape(-1, n)
        slack = 1e-6 * terms.abs().sum(0).cpu()               # fp32 accumulation, any order
        exact = terms.sum(0).cpu()
        assert ((got - want).abs() <= step * want.abs() + slack).all()
        # against the exact sum: the rounding to the tensor dtype and the quantizer's own (which on
        # bf16 tensors moves odd significands up) stack to at most two steps
        assert ((got - exact).abs() <= 2 * step * exact.abs() + slack).all()
        if spec.get("round") != "floor":                      # every result is a value of the format
            assert torch.equal(vec_quantize(got.to(dtype), mx_specs=specs).double(), got)


@pytest.mark.parametrize("op,mode", [(o, m) for o in ("add", "sub", "mul", "div")
                                     for m in ("tensor", "scalar_right", "scalar_left")] + [("recip", "scalar_left")])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("spec", [dict(bfloat=16), dict(bfloat=12, round="floor"), dict(fp=16, round="even")],
                         ids=["bfloat16", "bfloat12-floor", "fp16-even"])
def test_fused_vec_ops_equal_the_two_steps(dev, op, mode, dtype, spec):
    """vec_add / vec_sub / vec_mul / vec_div / vec_recip as one kernel against the same function on
    CPU tensors (torch's op, then the quantizer): bit for bit, special values included."""
    from microxcaling_amd import vector_ops as V
    from microxcaling_amd.specs import apply_mx_specs
    specs = _specs(**spec)
    g = torch.Generator().manual_seed(len(op) + len(mode))
    shape = (37, 131)                                              # 4847 elements: a ragged tail
    a = (torch.randn(*shape, generator=g) * torch.exp2(torch.randint(-30, 30, shape, generator=g).float())).to(dtype)
    b = (torch.randn(*shape, generator=g) * torch.exp2(torch.randint(-30, 30, shape, generator=g).float())).to(dtype)
    special = torch.tensor([0.0, -0.0, float("inf"), float("-inf"), float("nan"), 1e-39, 3e38, -3e38]).to(dtype)
    a[0, :8] = special
    b[0, :8] = special.flip(0)
    b[1, :8] = special
    fn = {"add": V.vec_add, "sub": V.vec_sub, "mul": V.vec_mul, "div": V.vec_div}.get(op)

    def run(x, y):
        if op == "recip":
            return V.vec_recip(x, mx_specs=specs)
        if mode == "tensor":
            return fn(x, y, mx_specs=specs)
        if mode == "scalar_right":
            return fn(x, 1.703125, mx_specs=specs)
        return fn(3, x, mx_specs=specs)
    want = run(a, b)
    with torch.no_grad():
        got = run(a.to(dev), b.to(dev))
    unfusable = dtype == torch.bfloat16 and spec.get("round") == "even"      # wide format, half-even, bf16 tensor
    assert (V._fused_binary(a.to(dev), b.to(dev), V._ADD, apply_mx_specs(specs), None) is None) == unfusable
    assert_bits_equal(got.cpu(), want, "%s %s" % (op, mode))


def test_layers_replay_from_a_hip_graph(dev):
    """The kernels take torch's current stream and allocate nothing themselves, so a block of MX
    layers can be captured once and replayed: linear (packed GEMM) -> GELU -> LayerNorm -> softmax.
    Every replay, with fresh input contents and eager work in between, must equal the eager result
    bit for bit."""
    from microxcaling_amd import activations as A, layernorm as L
    from microxcaling_amd.linear import linear
    from microxcaling_amd.softmax import softmax
    specs = _specs(w_elem_format="fp8_e4m3", a_elem_format="fp8_e4m3", block_size=32, bfloat=16)
    g = torch.Generator().manual_seed(5)
    w = (torch.randn(1024, 512, generator=g) * 0.05).to(torch.bfloat16).to(dev)
    b = torch.randn(1024, generator=g).to(torch.bfloat16).to(dev)
    ln = L.LayerNorm(1024, eps=1e-5, mx_specs=specs).to(torch.bfloat16).to(dev)

    def block(x):
        with torch.no_grad():
            h = linear(x, w, b, mx_specs=specs)
            h = A.gelu(h, mx_specs=specs)
            h = ln(h)
            return softmax(h, dim=-1, mx_specs=specs)

    static_x = torch.randn(512, 512, generator=g).to(torch.bfloat16).to(dev)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):                      # warm-up outside the capture (kernel attributes, caches)
        for _ in range(2):
            block(static_x)
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        static_y = block(static_x)
    for i in range(3):
        x = (torch.randn(512, 512, generator=g) * (i + 1)).to(torch.bfloat16).to(dev)
        want = block(x)                                # eager work between the replays
        torch.cuda.synchronize()
        static_x.copy_(x)
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(static_y.view(torch.int16), want.view(torch.int16)), i


def test_gemm_split_k_is_used_and_optional(dev):
    """Few output tiles: the library asks for a workspace and splits K; without one the product
    still comes out (unsplit), equal up to the order of the additions."""
    from microxcaling_amd import _lib
    from microxcaling_amd.fused import pack_mx, gemm_nt
    lib = _lib.gpu()
    assert lib.mxq_gemm_workspace_bytes(1, 64, 1024, 4096, 0) > 0
    assert lib.mxq_gemm_workspace_bytes(1, 4096, 4096, 4096, 0) == 0          # large-tile kernel
    assert lib.mxq_gemm_workspace_bytes(1, 64, 1024, 256, 0) == 0             # too few K steps
    g = torch.Generator().manual_seed(3)
    a, b = torch.randn(64, 4096, generator=g).to(dev), torch.randn(1024, 4096, generator=g).to(dev)
    (ac, asc, ak), (bc, bsc, bk) = pack_mx(a, "fp8_e4m3"), pack_mx(b, "fp8_e4m3")
    split = gemm_nt((ac, asc, ak), (bc, bsc, bk), torch.float32)
    plain = torch.empty_like(split)
    rc = lib.mxq_gemm_mx_nt(ac.data_ptr(), asc.data_ptr(), 0, bc.data_ptr(), bsc.data_ptr(), 0, None,
                            plain.data_ptr(), 0, 1, 64, 1024, 4096, 0, None, 0,
                            torch.cuda.current_stream().cuda_stream)
    assert rc == 0
    torch.cuda.synchronize()
    assert rel_err(split, plain) < 1e-4



@pytest.mark.parametrize("fmt", ["fp6_e2m3", "fp6_e3m2"])
@pytest.mark.parametrize("rnd", ["nearest", "floor", "even"])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_sixbit_pack_is_the_fake_quantized_tensor(dev, fmt, rnd, dtype):
    """fp6 elements as 6-bit codes (four in three bytes, little-endian bit stream): unpacking gives
    the oracle's _quantize_mx output bit for bit, for the row-wise and for the transposing pack, and
    the codes are those of the byte form."""
    from microxcaling_amd.fused import pack_mx, pack_mx_t, unpack_mx, CODES_E2M3, CODES_E3M2
    g = torch.Generator().manual_seed(78)
    x = torch.randn(96, 256, generator=g) * torch.exp(3 * torch.randn(96, 256, generator=g))
    x[3, 40] = float("inf")
    x[5, 70] = float("nan")
    x[7, :64] *= 1e-38
    x[9, :32] = 0.0
    x[11, :32] = -1e-30 * torch.rand(32, generator=g)
    x = x.to(dtype)
    want = O.quantize_mx(x, 8, fmt, axes=[-1], block_size=32, round=rnd)
    codes, scales, kind = pack_mx(x.to(dev), fmt, 8, rnd, nibbles=True)
    assert codes.shape == (96, 192) and scales.shape == (96, 8)
    assert kind == (CODES_E2M3 if fmt == "fp6_e2m3" else CODES_E3M2)
    assert_bits_equal(unpack_mx(codes, scales, kind, dtype), want, "6-bit codes")
    # the bit stream, decoded on the host, against the values of the byte codes at scale 1
    bytes_, scales8, kind8 = pack_mx(x.to(dev), fmt, 8, rnd)
    assert torch.equal(scales8, scales)
    elems = unpack_mx(bytes_, torch.full_like(scales8, 127), kind8, torch.float32).cpu()
    raw = codes.cpu().numpy().astype("uint64").reshape(96, 64, 3)
    word = raw[..., 0] | (raw[..., 1] << 8) | (raw[..., 2] << 16)                 # four elements per 24 bits
    import numpy as np
    c6 = torch.from_numpy(((word[..., None] >> (6 * np.arange(4, dtype="uint64"))) & 63).astype("int64")).reshape(96, 256)
    mant, bias = (3, 1) if fmt == "fp6_e2m3" else (2, 3)
    e, m, s = (c6 >> mant) & ((1 << (5 - mant)) - 1), c6 & ((1 << mant) - 1), (c6 >> 5) & 1
    val = torch.where(e > 0, ((1 << mant) + m).double() * torch.exp2((e - bias - mant).double()),
                      m.double() * 2.0 ** (1 - bias - mant))
    val = torch.where(s == 1, -val, val).float()
    finite = (scales8 != 255).repeat_interleave(32, dim=-1).cpu()
    assert torch.equal(val[finite], elems[finite])
    # transposing pack
    want_t = O.quantize_mx(x, 8, fmt, axes=[-2], block_size=32, round=rnd)
    codes, scales, kind = pack_mx_t(x.to(dev), fmt, 8, rnd, nibbles=True)
    assert codes.shape == (256, 72) and scales.shape == (256, 3)
    got = unpack_mx(codes, scales, kind, dtype).transpose(-1, -2).contiguous()
    assert_bits_equal(got, want_t, "6-bit codes, transposed")


def test_gemm_rejects_sixbit_codes(dev):
    """6-bit codes are a storage form: the GEMM says so instead of reading them as bytes."""
    from microxcaling_amd.fused import pack_mx, gemm_nt
    a = torch.randn(512, 512).to(dev)
    pa = pack_mx(a, "fp6_e2m3", nibbles=True)
    assert pa[0].shape == (512, 384)
    with pytest.raises(RuntimeError, match="6-bit codes are a storage form"):
        gemm_nt(pa, pa, torch.float32)
    with pytest.raises(RuntimeError, match="6-bit codes are a storage form"):
        gemm_nt(pack_mx(a, "fp6_e2m3"), pa, torch.float32)


@pytest.mark.skip(reason="the large-tile GEMM variant that read 6-bit codes was withdrawn: it was slower "
                         "than the same product on byte codes and a long run of it ended in a GPU memory "
                         "fault whose cause is not known")
@pytest.mark.parametrize("M,N,K,batch", [(2048, 4096, 1024, 1), (2050, 1800, 1152, 2), (4096, 2048, 512, 1),
                                         (530, 512, 640, 22)])
@pytest.mark.parametrize("fa,fb", [("fp6_e2m3", "fp6_e2m3"), ("fp6_e3m2", "fp6_e2m3"), ("fp6_e3m2", "fp6_e3m2")])
def test_fp6_gemm_on_sixbit_codes_against_fp64(dev, M, N, K, batch, fa, fb):
    """Both operands as 6-bit codes at the 4-bit MFMA rate: against fp64 on the unpacked operands,
    with a 2^-3 .. 2^3 spread of block scales, and against the same GEMM on byte codes."""
    from microxcaling_amd import _lib
    from microxcaling_amd.fused import pack_mx, unpack_mx, gemm_nt
    assert _lib.gpu().mxq_gemm_takes_sixbit(batch, M, N, K) == 1
    g = torch.Generator().manual_seed(M * 7 + N * 3 + K + batch)
    shape_a = (batch, M, K) if batch > 1 else (M, K)
    shape_b = (batch, N, K) if batch > 1 else (N, K)
    blk = lambda s: torch.exp2(torch.randint(-3, 4, s[:-1] + (s[-1] // 32, 1), generator=g).float())
    a = (torch.randn(*shape_a, generator=g).view(*shape_a[:-1], K // 32, 32) * blk(shape_a)).view(shape_a)
    b = (torch.randn(*shape_b, generator=g).view(*shape_b[:-1], K // 32, 32) * blk(shape_b)).view(shape_b)
    pa = pack_mx(a.to(dev), fa, nibbles=True)
    pb = pack_mx(b.to(dev), fb, nibbles=True)
    got = gemm_nt(pa, pb, torch.float32)
    qa = unpack_mx(*pa, torch.float32).double()
    qb = unpack_mx(*pb, torch.float32).double()
    want = qa @ qb.transpose(-1, -2)
    assert got.shape == want.shape
    assert rel_err(got, want) < 1e-3
    den = qa.abs() @ qb.abs().transpose(-1, -2)
    assert ((got.double() - want).abs() <= 2e-4 * den + 1e-30).all()
    on_bytes = gemm_nt(pack_mx(a.to(dev), fa), pack_mx(b.to(dev), fb), torch.float32)
    assert rel_err(got, on_bytes) < 1e-3
    from microxcaling_amd.elemwise_ops import _quantize_bfloat
    bias = torch.randn(N, generator=g).to(dev).to(torch.bfloat16)
    want16 = _quantize_bfloat(_quantize_bfloat(got.to(torch.bfloat16), 16, round="nearest") + bias, 16, round="nearest")
    got16 = gemm_nt(pa, pb, torch.bfloat16, bias=bias, epilogue_quant=True)
    assert torch.equal(got16.view(torch.int16), want16.view(torch.int16))
    with pytest.raises(RuntimeError, match="both operands"):
        gemm_nt(pa, pack_mx(b.to(dev), fb), torch.float32)


# ---- the plain-range shortcut of the bfloat16 quantizer against the general form ---------------------
def _general_form():
    """Context: the chain kernels never take the shortcut."""
    import contextlib
    from microxcaling_amd import custom_extensions as CE

    @contextlib.contextmanager
    def ctx():
        CE.set_general_form(True)
        try:
            yield
        finally:
            CE.set_general_form(False)
    return ctx()


def _edge_rows(rows, n, g, lo, hi):
    """bf16 rows that sit on the edges of a plain range [2^lo, 2^hi): both ends, alternating signs,
    constant rows (no spread at all), rows of two values one step apart, and random rows of every
    magnitude in between."""
    x = torch.randn(rows, n, generator=g) * torch.exp2(torch.randint(lo + 2, hi - 3, (rows, 1), generator=g).float())
    x[0] = 2.0 ** lo
    x[1] = -(2.0 ** lo)
    x[2] = 2.0 ** hi * (1 - 2.0 ** -8)
    x[3] = torch.where(torch.arange(n) % 2 == 0, 2.0 ** lo, -(2.0 ** hi) * (1 - 2.0 ** -8))
    x[4] = 1.0
    x[5] = torch.where(torch.arange(n) % 2 == 0, 1.0, 1.0 + 2.0 ** -7)
    x[6] = torch.where(torch.arange(n) % 3 == 0, 3.0, 2.0 ** lo)
    x[7] = torch.exp2(torch.linspace(lo, hi - 0.01, n)) * (1 - 2 * (torch.arange(n) % 2))
    x = x.to(torch.bfloat16)
    tiny = x.float().abs() < 2.0 ** lo
    x[tiny] = 2.0 ** lo
    x[x.float().abs() >= 2.0 ** hi] = 2.0 ** (hi - 1)
    return x


@pytest.mark.parametrize("n", [264, 2048, 8192, 16384])
@pytest.mark.parametrize("spec", [dict(bfloat=16), dict(bfloat=16, softmax_exp2=True),
                                  dict(bfloat=16, vec_use_exp2=True, vec_use_recip=True)])
def test_softmax_shortcut_equals_general_form(dev, n, spec):
    from microxcaling_amd.softmax import softmax
    g = torch.Generator().manual_seed(n)
    x = _edge_rows(24, n, g, -100, 100)
    x[8:16] = (torch.randn(8, n, generator=g) * 3).to(torch.bfloat16)     # ordinary logits
    # around the limits of the form without any special case: spreads of 83 .. 86 below the
    # maximum, smallest quotients next to the smallest normal number
    even = torch.arange(n) % 2 == 0
    x[16] = 1.0
    x[17] = torch.where(even, 1.0, -82.0).to(torch.bfloat16)
    x[18] = torch.where(even, 1.0, -83.5).to(torch.bfloat16)
    x[19] = torch.where(even, 1.0, -85.0).to(torch.bfloat16)
    x[20] = torch.where(torch.arange(n) == 5, 3.0, -80.0).to(torch.bfloat16)
    x[21] = torch.linspace(-80, 5, n).to(torch.bfloat16)
    x[22] = torch.where(torch.arange(n) < n // 2, 3.0, -75.0).to(torch.bfloat16)
    x[23] = torch.where(torch.arange(n) < 4, 2.0, -70.0).to(torch.bfloat16)
    x[x == 0] = 1.0
    specs = _specs(**spec)
    got = softmax(x.to(dev), dim=-1, mx_specs=specs).cpu()
    with _general_form():
        want = softmax(x.to(dev), dim=-1, mx_specs=specs).cpu()
    # The two forms quantize identically; rows whose inputs all lie within 85 of their maximum take the
    # hardware exponential in the shortcut (1 ulp, like expf, but not the same ulp), which the rounding
    # to bfloat16 lets through on about one element in 10^4: equal bit for bit on all but a few
    # elements (or the elements of a row whose sum moved), those one step of the format apart.
    same = got.view(torch.int16) == want.view(torch.int16)
    assert int((~same).any(-1).sum()) <= 2                 # rows with any difference (a changed row sum moves a whole row)
    d = (got.float() - want.float()).abs()
    assert bool((d <= 2 ** -6 * want.float().abs() + 2.0 ** -133).all())
    far = (x.float().max(-1, keepdim=True).values - x.float()).max(-1).values > 86     # rows outside that range
    assert torch.equal(got[far].view(torch.int16), want[far].view(torch.int16))


@pytest.mark.parametrize("layer", ["layernorm", "rmsnorm"])
@pytest.mark.parametrize("n", [264, 4096, 8192, 16384])
@pytest.mark.parametrize("eps", [1e-5, 1e-12, 0.0])
def test_norm_shortcut_equals_general_form(dev, layer, n, eps):
    """Inputs, weights and biases on the edges of their plain ranges, constant rows (variance 0:
    with eps = 0 the row scale is Inf and the wave must leave the shortcut), products that cancel
    the bias exactly, zero and negative-zero biases, weights of both signs."""
    from microxcaling_amd import layernorm as L
    from microxcaling_amd.specs import apply_mx_specs
    g = torch.Generator().manual_seed(n + len(layer))
    x = _edge_rows(40, n, g, -20, 20)
    w = torch.exp2(torch.linspace(-20, 19.99, n)) * (1 - 2 * (torch.arange(n) % 2).float())
    b = torch.randn(n, generator=g) * torch.exp2(torch.randint(-39, 39, (n,), generator=g).float())
    b = torch.sign(b) * b.abs().clamp(2.0 ** -39.5, 2.0 ** 39.5)
    b[::5] = 0.0
    w, b = w.to(torch.bfloat16), b.to(torch.bfloat16)
    specs = apply_mx_specs(_specs(bfloat=16))
    outs = []
    for wi, bi in ((w, b), (torch.ones_like(w), torch.zeros_like(b)), (-w, -b.abs())):
        for general in (False, True):
            if general:
                with _general_form():
                    r = L._fused_forward(x.to(dev), wi.to(dev), bi.to(dev), eps, specs, layer == "rmsnorm")
            else:
                r = L._fused_forward(x.to(dev), wi.to(dev), bi.to(dev), eps, specs, layer == "rmsnorm")
            assert r is not None
            outs.append([t.cpu() for t in r])
        for a, c, what in zip(outs[-2], outs[-1], ("output", "normalized input", "row statistic")):
            same = (a.view(torch.int16) == c.view(torch.int16)) | (torch.isnan(a) & torch.isnan(c))
            assert same.all(), what


@pytest.mark.parametrize("act", sorted(_ACTS))
@pytest.mark.parametrize("spec", [dict(bfloat=16), dict(bfloat=16, vec_use_exp2=True)], ids=["exp", "exp2"])
def test_activation_shortcut_equals_general_form(dev, act, spec):
    from microxcaling_amd import activations as A
    g = torch.Generator().manual_seed(len(act) + 1)
    x = _edge_rows(64, 2048, g, -20, 3).reshape(-1)
    specs = _specs(**spec)
    got = _ACTS[act](A, x.to(dev), specs).cpu()
    with _general_form():
        want = _ACTS[act](A, x.to(dev), specs).cpu()
    assert torch.equal(got.view(torch.int16), want.view(torch.int16))
    # every bf16 value of the range, both signs
    codes = torch.arange(0x3580, 0x4100, dtype=torch.int32)
    allv = torch.cat([codes, codes + 0x8000]).to(torch.int16).view(torch.bfloat16)
    allv = allv.repeat(2)[: (2 * allv.numel()) // 512 * 512]
    got = _ACTS[act](A, allv.to(dev), specs).cpu()
    with _general_form():
        want = _ACTS[act](A, allv.to(dev), specs).cpu()
    assert torch.equal(got.view(torch.int16), want.view(torch.int16))


@pytest.mark.parametrize("act", sorted(_ACTS))
@pytest.mark.parametrize("spec", [dict(bfloat=16), dict(bfloat=16, vec_use_exp2=True)], ids=["exp", "exp2"])
def test_activation_backward_shortcut_equals_general_form(dev, act, spec):
    """Saved tensors and gradients inside the plain ranges of the backward kernel (and a few waves
    outside: saturated sigmoids, large inputs), including the inputs around which the derivative of
    silu and gelu changes sign, where the last sum of the chain cancels."""
    from microxcaling_amd import activations as A
    g = torch.Generator().manual_seed(len(act) + 7)
    n = 512 * 400
    x = (torch.randn(n, generator=g) * 1.5).clamp(-5, 5)
    x[: 512 * 64] = torch.linspace(-1.5, -0.5, 512 * 64)          # the zeros of silu' and gelu'
    x[512 * 64: 512 * 72] = torch.linspace(5.0, 9.0, 512 * 8)     # saturating
    x[x.abs() < 2.0 ** -19] = 0.25
    x = x.to(torch.bfloat16)
    x[512 * 72: 512 * 80] = torch.linspace(-9.0, -4.0, 512 * 8)   # tiny logistic factors
    x = x.to(torch.bfloat16)
    grad = torch.randn(n, generator=g) * torch.exp2(torch.randint(-28, 38, (n,), generator=g).float())
    grad = (torch.sign(grad) * grad.abs().clamp(2.0 ** -29.5, 2.0 ** 39.5)).to(torch.bfloat16)
    grad[512 * 300:] = (grad[512 * 300:].float() * 2.0 ** -12).to(torch.bfloat16)     # partly below the range
    specs = _specs(**spec)
    grads = []
    for general in (False, True):
        xi = x.to(dev).requires_grad_(True)
        if general:
            with _general_form():
                _ACTS[act](A, xi, specs).backward(grad.to(dev))
        else:
            _ACTS[act](A, xi, specs).backward(grad.to(dev))
        grads.append(xi.grad.cpu())
    assert torch.equal(grads[0].view(torch.int16), grads[1].view(torch.int16))
    assert (grads[0].float() == 0).float().mean() < 0.2


@pytest.mark.parametrize("n", [264, 2048, 4096, 16384])
@pytest.mark.parametrize("spec", [dict(bfloat=16), dict(bfloat=16, softmax_exp2=True)], ids=["exp", "exp2"])
def test_softmax_backward_shortcut_equals_general_form(dev, n, spec):
    """Gradients and saved outputs inside the plain ranges (rows of ordinary logits), gradients on
    the edges of their range, a constant gradient (g - s cancels everywhere), rows with outputs that
    underflowed to zero and gradients outside the range (general form)."""
    from microxcaling_amd.softmax import softmax
    g = torch.Generator().manual_seed(n + 3)
    rows = 48
    x = (torch.randn(rows, n, generator=g) * 3).to(torch.bfloat16)
    x[40:44, ::7] = -200.0                                       # outputs that are exactly zero
    grad = torch.randn(rows, n, generator=g) * torch.exp2(torch.randint(-27, 27, (rows, 1), generator=g).float())
    grad[0] = 2.0 ** -30
    grad[1] = -(2.0 ** 30) * (1 - 2.0 ** -8)
    grad[2] = torch.where(torch.arange(n) % 2 == 0, 2.0 ** -30, 2.0 ** 29)
    grad[3] = 0.75
    grad[4] = torch.where(torch.arange(n) % 2 == 0, 1.0, 1.0 + 2.0 ** -7)
    grad[44:] = grad[44:] * 2.0 ** -40                           # below the range
    grad = torch.sign(grad) * grad.abs().clamp(min=2.0 ** -80)
    grad[:44] = torch.sign(grad[:44]) * grad[:44].abs().clamp(2.0 ** -30, 2.0 ** 29.9)
    grad = grad.to(torch.bfloat16)
    specs = _specs(**spec)
    grads = []
    for general in (False, True):
        xi = x.to(dev).requires_grad_(True)
        if general:
            with _general_form():
                softmax(xi, dim=-1, mx_specs=specs).backward(grad.to(dev))
        else:
            softmax(xi, dim=-1, mx_specs=specs).backward(grad.to(dev))
        grads.append(xi.grad.cpu())
    assert torch.equal(grads[0].view(torch.int16), grads[1].view(torch.int16))


@pytest.mark.parametrize("layer", ["layernorm", "rmsnorm"])
@pytest.mark.parametrize("n", [264, 4096, 16384])
def test_norm_backward_shortcut_equals_general_form(dev, layer, n):
    """Saved tensors of a forward pass over edge rows (constant rows: normalized input all +0),
    gradients on the edges of their range, rows whose projections cancel (gradient proportional to
    the normalized input, constant gradient), and rows outside the ranges."""
    from microxcaling_amd import layernorm as L
    from microxcaling_amd.specs import apply_mx_specs
    g = torch.Generator().manual_seed(n + 11)
    rms = layer == "rmsnorm"
    specs = apply_mx_specs(_specs(bfloat=16))
    x = _edge_rows(40, n, g, -20, 20)
    x[8:24] = torch.randn(16, n, generator=g).to(torch.bfloat16)
    w = (torch.exp2(torch.linspace(-20, 19.99, n)) * (1 - 2 * (torch.arange(n) % 2).float())).to(torch.bfloat16)
    for wi in (torch.ones_like(w), w):
        fwd = L._fused_forward(x.to(dev), wi.to(dev), torch.zeros_like(wi).to(dev), 1e-5, specs, rms)
        assert fwd is not None
        _, z, stat = fwd
        grad = torch.randn(40, n, generator=g) * torch.exp2(torch.randint(-27, 27, (40, 1), generator=g).float())
        grad[8] = 2.0 ** -30
        grad[9] = -(2.0 ** 30) * (1 - 2.0 ** -8)
        grad[10] = 0.5
        grad[11] = z[11].cpu().float()
        grad[12] = torch.where(torch.arange(n) % 2 == 0, 2.0 ** -30, -(2.0 ** 29))
        grad[:36] = torch.sign(grad[:36]) * grad[:36].abs().clamp(2.0 ** -30, 2.0 ** 29.9)
        grad[grad == 0] = 2.0 ** -30
        grad[36:] = grad[36:] * 2.0 ** -45                       # below the range
        grad = grad.to(torch.bfloat16).to(dev)
        got = L._fused_grad_input(grad, wi.to(dev), z, stat, specs, rms)
        with _general_form():
            want = L._fused_grad_input(grad, wi.to(dev), z, stat, specs, rms)
        assert got is not None and want is not None
        got, want = got.cpu(), want.cpu()
        same = (got.view(torch.int16) == want.view(torch.int16)) | (torch.isnan(got) & torch.isnan(want))
        assert same.all()
