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
