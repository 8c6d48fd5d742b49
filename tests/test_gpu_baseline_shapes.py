"""The benchmark configurations at their full sizes, through the kernel variants those sizes select,
against the CPU oracle on seeded samples (rows, columns or batches) of the same inputs.

  config 2   _quantize_mx, bf16 [8192, 8192] with outlier columns, fp6 / fp4, axes -1 and -2, three
             roundings: bit for bit on sampled rows and sampled columns
  config 3   _quantize_elemwise_core, fp32 [16384, 8192] of wide range with Inf / NaN / subnormals:
             bit for bit on sampled rows; reductions over axis 0 and -1 at [16384, 8192] (the axis-0
             kernel with eight column groups per lane): max exact, sum within 1e-5 * sum|x|
  config 4   mx.Linear forward, [16384, 4096] x [14336, 4096] + bias through linear(): the persistent
             256 x 256 tile kernel at K = 4096; fp32 tensors within 1e-3 (max |diff| / RMS), bf16
             tensors within one bf16 step of the product and of the sum on top of that
  config 5   mx.bmm Q.K^T [128, 2048, 128] MXFP6 e2m3 + bfloat16 softmax: sampled batches

The oracle only sees the samples (a few seconds of CPU work per case); the GPU runs the full
tensors."""
import numpy as np
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

ROUNDS = ["nearest", "floor", "even"]
BF16_MAX = 2 ** 127 * 255 / 128


@pytest.fixture(scope="module")
def dev():
    assert torch.cuda.is_available(), "these tests need a GPU"
    return torch.device("cuda:0")


def _specs(**kw):
    from microxcaling_amd.specs import finalize_mx_specs
    return finalize_mx_specs(dict(kw))


def _sample(n, count, seed, block=32):
    """Sorted sample of `count` indices below n: whole blocks of `block` neighbours (so that a
    sampled strip contains every member of its MX blocks), the first and the last block included."""
    g = torch.Generator().manual_seed(seed)
    nb = n // block
    picks = torch.randperm(nb, generator=g)[: max(count // block - 2, 0)].tolist()
    blocks = sorted(set(picks + [0, nb - 1]))
    return torch.cat([torch.arange(b * block, (b + 1) * block) for b in blocks])


# ---- config 2 -----------------------------------------------------------------------------------
@pytest.fixture(scope="module")
def outlier_tensor(dev):
    g = torch.Generator().manual_seed(7)
    x = torch.randn(8192, 8192, generator=g)
    idx = torch.randperm(8192, generator=g)[:81]
    scale = torch.ones(8192)
    scale[idx] = torch.exp(2.0 * torch.randn(81, generator=g))
    x = (x * scale).to(torch.bfloat16)
    return x, x.to(dev), idx


@pytest.mark.parametrize("fmt", ["fp6_e3m2", "fp6_e2m3", "fp4_e2m1"])
@pytest.mark.parametrize("axis", [-1, -2])
@pytest.mark.parametrize("rnd", ROUNDS)
def test_config2_full_size(dev, outlier_tensor, fmt, axis, rnd):
    from microxcaling_amd.mx_ops import _quantize_mx
    x, xd, outlier_cols = outlier_tensor
    got = _quantize_mx(xd, 8, fmt, axes=[axis], block_size=32, round=rnd)
    torch.cuda.synchronize()
    assert got.shape == x.shape and got.dtype == torch.bfloat16
    if axis == -1:
        # blocks lie inside a row: any set of rows is self-contained
        rows = _sample(8192, 512, 21, block=1)
        want = O.quantize_mx(x[rows].contiguous(), 8, fmt, axes=[-1], block_size=32, round=rnd)
        assert_bits_equal(got[rows.to(dev)].cpu(), want, "rows")
    else:
        # blocks lie inside a column: sampled columns (every outlier column among them), all rows
        cols = torch.unique(torch.cat([_sample(8192, 384, 22, block=1), outlier_cols]))
        want = O.quantize_mx(x[:, cols].contiguous(), 8, fmt, axes=[-2], block_size=32, round=rnd)
        assert_bits_equal(got[:, cols.to(dev)].cpu(), want, "columns")
    # everywhere: every block keeps a power-of-two scale, so |y| never exceeds 2 |x| + tiny and zeros stay zeros
    assert bool((got[xd == 0] == 0).all())
    assert bool(torch.isfinite(got).all())


# ---- config 3 -----------------------------------------------------------------------------------
def _wide_fp32(rows, cols, seed, specials=True):
    """randn * 10^U(-40, 40) computed in fp64 and cast to fp32 (values past the fp32 range become
    Inf by themselves), then 0.1 % of the positions set to +Inf / -Inf / NaN in turn and 1 % to random
    fp32 subnormals of either sign.  Built in slabs to bound the host memory."""
    g = torch.Generator().manual_seed(seed)
    out = torch.empty(rows, cols, dtype=torch.float32)
    step = 2048
    for r0 in range(0, rows, step):
        r1 = min(rows, r0 + step)
        v = torch.randn(r1 - r0, cols, generator=g, dtype=torch.float64)
        v *= 10.0 ** (torch.rand(r1 - r0, cols, generator=g, dtype=torch.float64) * 80 - 40)
        out[r0:r1] = v.to(torch.float32)
    flat = out.view(-1)
    n = flat.numel()
    if specials:
        k = n // 1000
        pos = torch.randint(0, n, (k,), generator=g)
        flat[pos] = torch.tensor([float("inf"), -float("inf"), float("nan")]).repeat(k // 3 + 1)[:k]
    m = n // 100
    pos = torch.randint(0, n, (m,), generator=g)
    sub = torch.randint(1, 1 << 23, (m,), generator=g, dtype=torch.int32)
    sub |= torch.randint(0, 2, (m,), generator=g, dtype=torch.int32) << 31
    flat[pos] = sub.view(torch.float32)
    return out


@pytest.fixture(scope="module")
def wide_tensor(dev):
    x = _wide_fp32(16384, 8192, 11)
    return x, x.to(dev)


@pytest.mark.parametrize("bits,ebits,max_norm", [(9, 8, BF16_MAX), (12, 5, 65504.0)])
@pytest.mark.parametrize("rnd", ["nearest", "even"])
@pytest.mark.parametrize("sat", [False, True])
def test_config3_elementwise_full_size(dev, wide_tensor, bits, ebits, max_norm, rnd, sat):
    from microxcaling_amd.elemwise_ops import _quantize_elemwise_core
    x, xd = wide_tensor
    got = _quantize_elemwise_core(xd, bits, ebits, max_norm, round=rnd, saturate_normals=sat)
    torch.cuda.synchronize()
    rows = _sample(16384, 256, 31, block=1)
    want = O.quantize_elemwise_core(x[rows].clone(), bits, ebits, max_norm, round=rnd, saturate_normals=sat)
    assert_bits_equal(got[rows.to(dev)].cpu(), want, "sampled rows")
    # the whole output: idempotent (a quantized tensor is a fixed point of its quantizer), and Inf / NaN
    # of the input where they were
    again = _quantize_elemwise_core(got, bits, ebits, max_norm, round=rnd, saturate_normals=sat)
    fin = torch.isfinite(got)
    assert bool(torch.equal(again[fin], got[fin]))
    # NaN exactly where the input has one -- except in the last 64 steps below the largest fp32 number,
    # where the reference's floor(log2(x)) comes out as 128 and 2^128 turns the element into NaN
    # (mx/elemwise_ops.py:135-141; a handful of the 134 million elements land there)
    zone = xd.abs() >= torch.tensor(0x7F7FFFC0, dtype=torch.int32).view(torch.float32).item()
    new_nan = torch.isnan(got) & ~torch.isnan(xd)
    assert bool((new_nan <= (zone & torch.isfinite(xd))).all())
    assert bool((torch.isnan(got) | ~torch.isnan(xd)).all())
    assert bool((torch.isinf(got) | ~torch.isinf(xd)).all())


def _check_sum(got, x, dim):
    """fp32 sum against an fp64 sum: NaN where IEEE addition gives NaN (a NaN, or Inf of both signs),
    +-Inf where it gives Inf, else within 1e-5 * sum |x|."""
    ref = x.double().sum(dim)
    got = got.double()
    assert bool(torch.equal(torch.isnan(got), torch.isnan(ref)))
    inf = torch.isinf(ref)
    assert bool(torch.equal(got[inf], ref[inf]))
    fin = torch.isfinite(ref)
    tol = 1e-5 * torch.where(torch.isfinite(x), x, torch.zeros_like(x)).double().abs().sum(dim)
    assert bool(((got[fin] - ref[fin]).abs() <= tol[fin]).all())
    return int(fin.sum()), int(inf.sum()), int(torch.isnan(ref).sum())


@pytest.fixture(scope="module")
def reduce_tensor(dev):
    """Wide range, but |x| <= 1e30 so that fp32 partial sums cannot overflow where the fp64 sum does
    not; +-Inf / NaN confined to a tenth of the rows and a tenth of the columns, so that both
    reductions see finite, Inf and NaN results."""
    g = torch.Generator().manual_seed(13)
    x = torch.empty(16384, 8192)
    for r0 in range(0, 16384, 2048):
        v = torch.randn(2048, 8192, generator=g)
        v *= 10.0 ** (torch.rand(2048, 8192, generator=g) * 60 - 30)
        x[r0:r0 + 2048] = v
    rr = torch.randint(0, 16384, (1600,), generator=g)
    cc = torch.randint(0, 8192, (1600,), generator=g) // 10 * 10
    x[rr // 10 * 10, cc] = torch.tensor([float("inf"), -float("inf"), float("nan")]).repeat(534)[:1600]
    return x, x.to(dev)


def test_config3_reductions_full_size(dev, reduce_tensor):
    from microxcaling_amd.custom_extensions import funcs
    x, xd = reduce_tensor
    xg = xd.double()
    for dim, fsum, fmax in ((0, funcs.reduce_sum_outer_dim, funcs.reduce_max_outer_dim),
                            (-1, funcs.reduce_sum_inner_dim, funcs.reduce_max_inner_dim)):
        s = fsum(xd)
        m = fmax(xd)
        torch.cuda.synchronize()
        counts = _check_sum(s, xg, dim)
        assert min(counts) > 0, counts                          # all three classes occur
        assert_bits_equal(m.cpu(), torch.max(x, dim=dim).values, "max over axis %d" % dim)


@pytest.mark.parametrize("shape", [(256, 8192), (256, 4096), (4100, 12288), (33, 8200)])
def test_outer_reduction_with_eight_and_four_column_groups_per_lane(dev, shape):
    """Rows of >= 8192 (>= 4096) columns take the axis-0 kernel instance with eight (four) groups of
    four columns per lane; 12288 and 8200 columns leave the last workgroup partly empty."""
    from microxcaling_amd.custom_extensions import funcs
    g = torch.Generator().manual_seed(shape[0] + shape[1])
    x = torch.randn(*shape, generator=g) * 10.0 ** (torch.rand(*shape, generator=g) * 20 - 10)
    x[3, 5] = float("nan")
    x[7, shape[1] - 3] = float("inf")
    xd = x.to(dev)
    _check_sum(funcs.reduce_sum_outer_dim(xd), xd.double(), 0)
    assert_bits_equal(funcs.reduce_max_outer_dim(xd).cpu(), torch.max(x, dim=0).values, "max")


# ---- config 4 -----------------------------------------------------------------------------------
M4, N4, K4 = 16384, 14336, 4096


@pytest.fixture(scope="module")
def linear_operands():
    g = torch.Generator().manual_seed(4)
    x = torch.randn(M4, K4, generator=g)
    w = torch.randn(N4, K4, generator=g) * 0.02
    b = torch.randn(N4, generator=g)
    return x, w, b


def _plan(batch, M, N, K, kind=0):
    from microxcaling_amd import _lib
    return _lib.gpu().mxq_gemm_plan(batch, M, N, K, kind)


@pytest.mark.parametrize("case", ["fp8_bf16", "fp8_f32", "fp4_bf16", "fp8_bf16_bfloat16", "fp6_bf16_nobias"])
def test_config4_full_size_linear(dev, linear_operands, case):
    from microxcaling_amd.linear import linear
    fmt = {"fp8": "fp8_e4m3", "fp4": "fp4_e2m1", "fp6": "fp6_e2m3"}[case.split("_")[0]]
    dtype = torch.float32 if "_f32" in case else torch.bfloat16
    bfloat = 16 if case.endswith("bfloat16") else 0
    x, w, b = (t.to(dtype) for t in linear_operands)
    if case.endswith("nobias"):
        b = None
    # the shape must take the persistent 256 x 256 tile kernel (e2m1 nibbles when both operands are fp4)
    assert _plan(1, M4, N4, K4, 4 if fmt == "fp4_e2m1" else 0) == 2
    specs = _specs(w_elem_format=fmt, a_elem_format=fmt, block_size=32, bfloat=bfloat)
    got = linear(x.to(dev), w.to(dev), None if b is None else b.to(dev), mx_specs=specs)
    torch.cuda.synchronize()
    assert got.shape == (M4, N4) and got.dtype == dtype
    # 256 sampled rows, among them the first and last rows of the first and last tile rows
    rows = torch.unique(torch.cat([_sample(M4, 224, 41, block=1), torch.tensor([0, 255, 256, M4 - 256, M4 - 1])]))
    want = O.mx_linear_forward(x[rows].contiguous(), w, b, fmt, fmt, bfloat=bfloat).float()
    have = got[rows.to(dev)].float().cpu()
    diff = (have - want).abs()
    rms = want.pow(2).mean().sqrt()
    if dtype == torch.float32:
        assert (diff.max() / rms).item() < 1e-3
    else:
        # bf16 tensors round the product and then the sum with the bias to bf16 (and, with bfloat = 16,
        # quantize both): one bf16 step of the larger of the two on top of the accumulation tolerance
        # (with bfloat = 16 the quantizer keeps even significands only, and the product's step carries
        # over into the sum: |product| <= |sum| + |bias|)
        mag = (2 if bfloat else 1) * want.abs() + (0 if b is None else b.float().abs().view(1, -1))
        assert bool((diff <= 2 ** -6 * mag + 2e-3 * rms).all()), (diff.max().item(), rms.item())
        # and the bulk is far closer than that bound: the mean difference stays below a tenth of a step
        assert (diff / (2 ** -8 * mag + 1e-30)).mean().item() < 0.25
    assert bool(torch.isfinite(got).all())


def test_config4_rows_do_not_depend_on_their_tile(dev, linear_operands):
    """The same 256 activations placed at the start, in the middle and at the end of the [16384, 4096]
    input give bit-identical output rows (different workgroups, tile rows and K-walk starting points)."""
    from microxcaling_amd.linear import linear
    x, w, b = (t.to(torch.bfloat16) for t in linear_operands)
    x = x.clone()
    x[8192 + 100:8192 + 356] = x[:256]
    x[M4 - 256:] = x[:256]
    specs = _specs(w_elem_format="fp8_e4m3", a_elem_format="fp8_e4m3", block_size=32)
    got = linear(x.to(dev), w.to(dev), b.to(dev), mx_specs=specs)
    torch.cuda.synchronize()
    first = got[:256].view(torch.int16)
    assert bool(torch.equal(got[8192 + 100:8192 + 356].view(torch.int16), first))
    assert bool(torch.equal(got[M4 - 256:].view(torch.int16), first))


# ---- config 5 -----------------------------------------------------------------------------------
def test_config5_full_size_bmm_softmax(dev):
    from microxcaling_amd.bmm import bmm
    from microxcaling_amd.softmax import softmax
    g = torch.Generator().manual_seed(5)
    B, S, D = 128, 2048, 128
    q = torch.randn(B, S, D, generator=g).to(torch.bfloat16)
    k = torch.randn(B, S, D, generator=g).to(torch.bfloat16)
    specs = _specs(a_elem_format="fp6_e2m3", block_size=32, bfloat=16)
    logits = bmm(q.to(dev), k.to(dev).transpose(-1, -2), mx_specs=specs)
    probs = softmax(logits, dim=-1, mx_specs=specs)
    # the same in one launch (logits in registers): what the benchmark times
    from microxcaling_amd.bmm import bmm_softmax
    fused_probs = bmm_softmax(q.to(dev), k.to(dev).transpose(-1, -2), mx_specs=specs)
    torch.cuda.synchronize()
    assert logits.shape == (B, S, S) and probs.dtype == torch.bfloat16
    for bz in (0, 63, 127):
        want = O.mx_bmm_forward(q[bz:bz + 1], k[bz:bz + 1].transpose(-1, -2), "fp6_e2m3", bfloat=16)
        have = logits[bz:bz + 1].cpu()
        # the logits are re-rounded to bfloat16: one step of the format where the fp32 sums differ in order
        d = (have.float() - want.float()).abs()
        assert bool((d <= 2 ** -7 * want.float().abs() + 1e-3 * want.float().pow(2).mean().sqrt()).all())
        assert (d > 0).float().mean().item() < 0.05, (d > 0).float().mean().item()
        # the softmax of the logits the GPU produced, against the oracle's chain on those same logits
        sm_want = O.softmax_forward(have, -1, bfloat=16).float()
        sm = probs[bz:bz + 1].float().cpu()
        assert (sm - sm_want).abs().max().item() <= 2 ** -8
        assert ((sm - sm_want).abs() > 0).float().mean().item() < 0.02, ((sm - sm_want).abs() > 0).float().mean().item()
        fd = (fused_probs[bz:bz + 1].float().cpu() - sm_want).abs()
        assert bool((fd <= 2 ** -6 * sm_want + 2.0 ** -132).all()) and (fd > 0).float().mean().item() < 0.02, \
            (fd.max().item(), (fd > 0).float().mean().item())
    # every row of probabilities sums to one within the quantization of 2048 bfloat16 terms
    for p_ in (probs, fused_probs):
        sums = p_.float().sum(-1)
        assert bool(((sums - 1).abs() < 0.02).all())
