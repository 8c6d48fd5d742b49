"""Linear layers that keep their weight as MX codes only (prequantize_weights(keep_dense=False)), and
the bias-only gradient of linear().  The GPU cases check the packed form through the fused GEMM (C ABI);
the CPU cases what the module does around it: loading a saved state, refusing inputs it cannot serve."""
import pytest
import torch

from helpers import assert_bits_equal
from oracle import mx_oracle as O


def _specs(**kw):
    from microxcaling_amd.specs import finalize_mx_specs
    return finalize_mx_specs(dict(kw), early_exit=False)


def test_a_codes_only_state_loads_into_a_fresh_layer_and_refuses_cpu_inputs():
    from microxcaling_amd.linear import Linear
    N, K = 64, 128
    specs = _specs(w_elem_format="fp8_e4m3", a_elem_format="fp8_e4m3", block_size=32, bfloat=16, round="even")
    g = torch.Generator().manual_seed(5)
    state = {"weight": torch.empty(0, dtype=torch.bfloat16),
             "bias": torch.randn(N, generator=g).to(torch.bfloat16),
             "weight_codes": torch.randint(0, 255, (N, K), generator=g, dtype=torch.uint8),
             "weight_scales": torch.randint(100, 140, (N, K // 32), generator=g, dtype=torch.uint8),
             "weight_code_kind": torch.tensor(0, dtype=torch.int32)}
    lin = Linear(K, N, mx_specs=specs).eval()
    lin.load_state_dict(state)                                  # strict: every key finds its place
    assert lin.prequantized_weights and lin.weight.numel() == 0 and lin.bias.dtype == torch.bfloat16
    assert lin.packed_weight_bytes() == N * K + N * K // 32
    saved = lin.state_dict()
    assert torch.equal(saved["weight_codes"], state["weight_codes"]) and int(saved["weight_code_kind"]) == 0
    with pytest.raises(RuntimeError, match="dropped its dense weight"):
        lin(torch.randn(4, K).to(torch.bfloat16))               # CPU input: only the fused GEMM reads codes
    with pytest.raises(RuntimeError, match="dropped already"):
        lin.prequantize_weights()


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_bias_only_gradient_on_cpu(dtype):
    """linear() when only the bias wants a gradient (mx/linear.py:187-196): grad_bias is the quantized
    column sum of the quantized output gradient, the other two gradients are not computed."""
    from microxcaling_amd.linear import linear
    specs = _specs(w_elem_format="fp6_e3m2", a_elem_format="fp6_e3m2", block_size=32, bfloat=16)
    g = torch.Generator().manual_seed(8)
    x, w = torch.randn(3, 40, 64, generator=g).to(dtype), torch.randn(96, 64, generator=g).to(dtype)
    b = torch.randn(96, generator=g).to(dtype).requires_grad_(True)
    go = torch.randn(3, 40, 96, generator=g).to(dtype)
    y = linear(x, w, b, mx_specs=specs)
    y.backward(go)
    want = O.mx_linear_backward(x, w, go, True, "fp6_e3m2", bfloat=16)[2]
    assert_bits_equal(b.grad, want, "grad_bias")
    assert_bits_equal(y.detach(), O.mx_linear_forward(x, w, b.detach(), "fp6_e3m2", "fp6_e3m2", bfloat=16), "output")


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_bias_only_gradient_on_the_gpu(dtype):
    """The same on the GPU, where the forward pass may leave the operands' quantization to the pack
    kernels because neither operand keeps a gradient: bias gradient bit for bit (a sum of quantized
    values in torch's order is not promised, so: within one step of the format), output within the
    tolerance of the fused GEMM."""
    from microxcaling_amd.linear import linear
    assert torch.cuda.is_available(), "this test needs a GPU"
    dev = torch.device("cuda:0")
    specs = _specs(w_elem_format="fp8_e4m3", a_elem_format="fp8_e4m3", block_size=32, bfloat=16, custom_cuda=True)
    g = torch.Generator().manual_seed(9)
    x, w = torch.randn(2, 256, 512, generator=g).to(dtype), torch.randn(384, 512, generator=g).to(dtype)
    b0 = torch.randn(384, generator=g).to(dtype)
    go = torch.randn(2, 256, 384, generator=g).to(dtype)
    b = b0.to(dev).requires_grad_(True)
    y = linear(x.to(dev), w.to(dev), b, mx_specs=specs)
    y.backward(go.to(dev))
    torch.cuda.synchronize()
    want_b = O.mx_linear_backward(x, w, go, True, "fp8_e4m3", bfloat=16)[2].float()
    got_b = b.grad.float().cpu()
    assert b.grad.dtype == dtype and bool((got_b - want_b).abs().le(2 ** -7 * want_b.abs() + 1e-6).all())
    ref = O.mx_linear_forward(x, w, b0, "fp8_e4m3", "fp8_e4m3", bfloat=16).float()
    diff = (y.detach().float().cpu() - ref).abs()
    assert bool((diff <= 2 ** -6 * (ref.abs() + b0.float().abs()) + 2e-3 * ref.pow(2).mean().sqrt()).all())


@pytest.mark.gpu
def test_a_codes_only_layer_moves_saves_and_reloads_on_the_gpu():
    """prequantize_weights(keep_dense=False) on the GPU: the codes are buffers of the module, so
    state_dict() carries them, a fresh layer loads them and gives the same outputs bit for bit, moving
    the layer to the CPU makes it refuse (instead of multiplying an empty weight), moving it back
    serves again; an fp32 input is refused with the same message."""
    from microxcaling_amd.linear import Linear
    assert torch.cuda.is_available(), "this test needs a GPU"
    dev = torch.device("cuda:0")
    M, N, K = 256, 384, 512
    specs = _specs(w_elem_format="fp8_e4m3", a_elem_format="fp8_e4m3", block_size=32, bfloat=16, round="even",
                   custom_cuda=True)
    torch.manual_seed(21)
    lin = Linear(K, N, mx_specs=specs).to(dev).eval()
    x = torch.randn(M, K, generator=torch.Generator().manual_seed(22)).to(torch.bfloat16).to(dev)
    lin.prequantize_weights(keep_dense=False)
    with torch.no_grad():
        first = lin(x)
    assert lin.weight.numel() == 0 and lin.packed_weight_bytes() == N * K + N * K // 32
    state = {k: v.clone() for k, v in lin.state_dict().items()}
    assert {"weight_codes", "weight_scales", "weight_code_kind"} <= set(state)
    fresh = Linear(K, N, mx_specs=specs).to(dev).eval()
    fresh.load_state_dict(state)
    with torch.no_grad():
        assert torch.equal(fresh(x).view(torch.int16), first.view(torch.int16))
        with pytest.raises(RuntimeError, match="dropped its dense weight"):
            lin(x.float())
        lin.cpu()
        if x.device.type == "cuda":                     # (a dry run on CPU tensors has one device only)
            with pytest.raises(RuntimeError, match="dropped its dense weight"):
                lin(x)
        lin.to(dev)
        assert torch.equal(lin(x).view(torch.int16), first.view(torch.int16))
