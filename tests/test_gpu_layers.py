"""Normalization layers and activations on the GPU against the same layers on CPU tensors (which
tests/test_layer_golden.py pins bit for bit to the reference's own layers).  Every step of these
chains is a torch pointwise / reduction op followed by the HIP elementwise quantizer; exp, tanh and
the order of the reductions differ in the last bit between the devices, which the quantizer can
turn into one step of bfloat16: tolerance one part in 2^7 of the largest value, and at most 2 % of
the elements different at all."""
import pytest
import torch

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def dev():
    assert torch.cuda.is_available(), "GPU tests need a GPU"
    from microxcaling_amd import _lib
    _lib.gpu()
    return torch.device("cuda:0")


def _specs(**kw):
    from microxcaling_amd.specs import finalize_mx_specs
    return finalize_mx_specs(dict(kw))


def _near(got, want, what):
    got, want = got.detach().float().cpu(), want.detach().float()
    assert got.shape == want.shape, what
    diff = (got - want).abs()
    assert diff.max().item() <= 2.0 ** -7 * want.abs().max().item(), (what, diff.max().item())
    assert (diff > 0).float().mean().item() <= 0.02, (what, (diff > 0).float().mean().item())


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("layer", ["layernorm", "rmsnorm"])
def test_norm_layers(dev, dtype, layer):
    from microxcaling_amd.layernorm import LayerNorm, RMSNorm
    cls = {"layernorm": LayerNorm, "rmsnorm": RMSNorm}[layer]
    specs = _specs(bfloat=16, quantize_backprop=True)
    g = torch.Generator().manual_seed(5)
    x = (torch.randn(6, 40, 256, generator=g) * 2 + 0.3).to(dtype)
    go = torch.randn(6, 40, 256, generator=g).to(dtype)
    ref = cls(256, eps=1e-5, mx_specs=specs).to(dtype)
    with torch.no_grad():
        ref.weight.copy_(torch.randn(256, generator=g))
        ref.bias.copy_(torch.randn(256, generator=g))
    gpu = cls(256, eps=1e-5, mx_specs=specs).to(dtype)
    gpu.load_state_dict(ref.state_dict())
    gpu.to(dev)
    xc, xg = x.clone().requires_grad_(True), x.to(dev).requires_grad_(True)
    oc, og = ref(xc), gpu(xg)
    oc.backward(go)
    og.backward(go.to(dev))
    _near(og, oc, "forward")
    _near(xg.grad, xc.grad, "grad_input")
    _near(gpu.weight.grad, ref.weight.grad, "grad_weight")
    _near(gpu.bias.grad, ref.bias.grad, "grad_bias")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("name", ["sigmoid", "tanh", "relu", "relu6", "leaky_relu", "silu", "gelu", "gelu1"])
def test_activations(dev, dtype, name):
    from microxcaling_amd import activations as act
    specs = _specs(bfloat=16, quantize_backprop=True)
    fn = {"sigmoid": lambda t: act.sigmoid(t, mx_specs=specs), "tanh": lambda t: act.tanh(t, mx_specs=specs),
          "relu": lambda t: act.relu(t, mx_specs=specs), "relu6": lambda t: act.relu6(t, mx_specs=specs),
          "leaky_relu": lambda t: act.leaky_relu(t, 0.1, mx_specs=specs),
          "silu": lambda t: act.silu(t, mx_specs=specs), "gelu": lambda t: act.gelu(t, mx_specs=specs),
          "gelu1": lambda t: act.gelu(t, mx_specs=specs, first_order_gelu=True)}[name]
    g = torch.Generator().manual_seed(6)
    x = (torch.randn(64, 512, generator=g) * 3).to(dtype)
    go = torch.randn(64, 512, generator=g).to(dtype)
    xc, xg = x.clone().requires_grad_(True), x.to(dev).requires_grad_(True)
    oc, og = fn(xc), fn(xg)
    oc.backward(go)
    og.backward(go.to(dev))
    _near(og, oc, "forward")
    _near(xg.grad, xc.grad, "backward")


def _run_both(dev, make, x, go, loose=False):
    """The same module on the CPU and on the GPU (same parameters), forward and backward."""
    torch.manual_seed(0)
    ref = make()
    gpu = make()
    gpu.load_state_dict(ref.state_dict())
    gpu.to(dev)
    xc, xg = x.clone().requires_grad_(True), x.to(dev).requires_grad_(True)
    oc, og = ref(xc), gpu(xg)
    if isinstance(oc, tuple):
        oc, og = oc[0], og[0]
    oc.backward(go)
    og.backward(go.to(dev))
    near = _near_loose if loose else _near
    near(og, oc, "forward")
    near(xg.grad, xc.grad, "grad_input")
    for (n, pc), (_, pg) in zip(ref.named_parameters(), gpu.named_parameters()):
        near(pg.grad, pc.grad, "grad " + n)


def _near_loose(got, want, what):
    """Contractions (MIOpen / hipBLASLt vs the CPU's order of summation) followed by a bfloat16
    quantizer: one bfloat16 step of the largest value, a tenth of the elements may differ."""
    got, want = got.detach().float().cpu(), want.detach().float()
    assert got.shape == want.shape, what
    diff = (got - want).abs()
    assert diff.max().item() <= 2.0 ** -6 * want.abs().max().item(), (what, diff.max().item())
    assert (diff > 0).float().mean().item() <= 0.10, (what, (diff > 0).float().mean().item())


def test_convolutions(dev):
    from microxcaling_amd.convolution import Conv2d
    s = _specs(w_elem_format="fp8_e4m3", a_elem_format="fp8_e4m3", block_size=32, bfloat=16,
               quantize_backprop=True)
    g = torch.Generator().manual_seed(8)
    x = torch.randn(4, 64, 12, 12, generator=g)
    _run_both(dev, lambda: Conv2d(64, 96, 3, stride=2, padding=1, mx_specs=s), x,
              torch.randn(4, 96, 6, 6, generator=g), loose=True)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("layer", ["layernorm", "rmsnorm"])
@pytest.mark.parametrize("shape", [(64, 4096), (5, 7, 1000), (33, 264), (9, 8), (5, 8192), (3, 16384)])
@pytest.mark.parametrize("spec", [dict(bfloat=16), dict(bfloat=16, round="floor"), dict(fp=16),
                                  dict(bfloat=16, round="even")])
def test_fused_norm_kernel_against_the_separate_steps(dev, dtype, layer, shape, spec):
    """mxq_norm_lastdim vs the chain of vector ops it replaces, both on the GPU (set_fused switches
    between them): output, saved normalized input, row statistic and gradients.  Only the order of
    the two row sums differs."""
    from microxcaling_amd import gemm
    from microxcaling_amd.layernorm import LayerNorm, RMSNorm, _fused_forward
    cls = {"layernorm": LayerNorm, "rmsnorm": RMSNorm}[layer]
    specs = _specs(quantize_backprop=True, **spec)
    g = torch.Generator().manual_seed(sum(shape))
    x = (torch.randn(*shape, generator=g) * 2 + 0.3).to(dtype)
    if "fp" in spec and shape[-1] > 4096:
        x = x * 0.25                                   # keep the row sums inside the fp16 format's range
    go = torch.randn(*shape, generator=g).to(dtype)
    m = cls(shape[-1], eps=1e-5, mx_specs=specs).to(dtype)
    with torch.no_grad():
        m.weight.copy_(torch.randn(shape[-1], generator=g))
        m.bias.copy_(torch.randn(shape[-1], generator=g))
    m.to(dev)
    res = []
    for fused in (True, False):
        gemm.set_fused(fused)
        try:
            xi = x.to(dev).requires_grad_(True)
            m.zero_grad()
            out = m(xi)
            out.backward(go.to(dev))
            res.append((out.detach().cpu(), xi.grad.cpu(), m.weight.grad.cpu().clone(), m.bias.grad.cpu().clone()))
        finally:
            gemm.set_fused(True)
    for got, want, what in zip(res[0], res[1], ("forward", "grad_input", "grad_weight", "grad_bias")):
        _near(got, want, what)


def test_layers_with_dither_rounding(dev):
    """mx_specs['round'] = 'dither': the kernels that run a whole chain of steps decline (each step
    needs its own noise), the layers run their separate steps with the dither kernels, forward and
    backward; results stay within the formats' steps of the round-to-nearest ones."""
    from microxcaling_amd.activations import gelu
    from microxcaling_amd.layernorm import LayerNorm
    from microxcaling_amd.linear import Linear
    from microxcaling_amd.softmax import softmax
    g = torch.Generator().manual_seed(8)
    x = torch.randn(64, 256, generator=g).to(torch.bfloat16).to(dev)
    out = {}
    for rnd in ("nearest", "dither"):
        specs = _specs(w_elem_format="fp8_e4m3", a_elem_format="fp8_e4m3", block_size=32, bfloat=16, round=rnd)
        torch.manual_seed(1)
        lin = Linear(256, 128, mx_specs=specs).to(torch.bfloat16).to(dev)
        ln = LayerNorm(128, eps=1e-5, mx_specs=specs).to(torch.bfloat16).to(dev)
        xi = x.clone().requires_grad_(True)
        y = softmax(gelu(ln(lin(xi)), mx_specs=specs), dim=-1, mx_specs=specs)
        (y * torch.arange(128, device=dev).to(torch.bfloat16)).sum().backward()
        assert torch.isfinite(y).all() and torch.isfinite(xi.grad).all() and torch.isfinite(lin.weight.grad).all()
        out[rnd] = (y.detach().float(), xi.grad.float())
    assert (out["dither"][0] - out["nearest"][0]).abs().max().item() <= 0.05
    assert (out["dither"][0].sum(-1) - 1).abs().max().item() <= 0.05
    assert not torch.equal(out["dither"][0], out["nearest"][0])
