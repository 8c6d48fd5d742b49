"""MX linear layer: same interface as the reference's mx/linear.py."""
import torch
import torch.nn.functional as F

from .elemwise_ops import quantize_elemwise_op
from .gemm import (inputs_can_skip_bfloat16_pass, mx_grad_contract, mx_linear_contract,
                   pack_can_quantize_first)
from .mx_ops import quantize_mx_op
from .specs import apply_mx_specs, get_backwards_mx_specs, mx_assert_test

f_linear = F.linear
torch_matmul = torch.matmul      # the stock function: inject_pyt_ops rebinds torch.matmul later


class LinearFunction(torch.autograd.Function):
    """Forward (mx/linear.py:20-101): bfloat-quantize input / weight / bias, MX-quantize both
    operands along the input-feature axis, multiply, bfloat-quantize, add the bias, bfloat-quantize.
    Backward (mx/linear.py:103-200): the two gradient products with their operands MX-quantized
    along the axis being contracted."""

    @staticmethod
    def forward(ctx, input, weight, bias=None, mx_specs=None, prequantized_weights=False,
                name=None, packed_weight=None):
        # inference (no gradient wanted for input, weight or bias, so backward never runs and nothing
        # keeps the quantized operands): their bfloat16 quantization is left to the
        # pack kernels of the fused GEMM (prequantized weights imply round-half-even, where that
        # quantization is a cast and there is nothing to leave)
        if not prequantized_weights and \
                inputs_can_skip_bfloat16_pass(ctx.needs_input_grad[:3], (input, weight), mx_specs,
                                              mx_specs["round_output"]) and \
                pack_can_quantize_first(mx_specs, mx_specs["round_weight"]):
            bf_bias = None if bias is None else quantize_elemwise_op(
                bias, mx_specs=mx_specs, round=mx_specs["round_weight"])
            output, finished = mx_linear_contract(input, weight, mx_specs["a_elem_format"],
                                                  mx_specs["w_elem_format"], mx_specs,
                                                  mx_specs["round_mx_output"],
                                                  out_round=mx_specs["round_output"], bias=bf_bias,
                                                  pre_bfloat16=True)
            if output is not None:
                if not finished:
                    output = quantize_elemwise_op(output, mx_specs=mx_specs, round=mx_specs["round_output"])
                    if bias is not None:
                        output = quantize_elemwise_op(output + bf_bias, mx_specs=mx_specs,
                                                      round=mx_specs["round_output"])
                ctx.has_bias = bias is not None
                ctx.mx_specs = get_backwards_mx_specs(mx_specs)
                ctx.prequantized_weights = prequantized_weights
                ctx.name = name
                return output
        bf_in = quantize_elemwise_op(input, mx_specs=mx_specs, round=mx_specs["round_output"])
        if prequantized_weights:
            assert weight.dtype == torch.bfloat16
            assert bias is None or bias.dtype == torch.bfloat16
            bf_weight, bf_bias = weight, bias
        else:
            bf_weight = quantize_elemwise_op(weight, mx_specs=mx_specs,
                                             round=mx_specs["round_weight"])
            bf_bias = None if bias is None else quantize_elemwise_op(
                bias, mx_specs=mx_specs, round=mx_specs["round_weight"])
        ctx.has_bias = bias is not None
        if mx_specs["quantize_backprop"]:
            ctx.save_for_backward(bf_in, bf_weight)
        else:
            ctx.save_for_backward(input, weight)

        # the steps after the product -- quantize, add the bias, quantize -- ride in the fused
        # GEMM's epilogue when the quantizer allows it (finished)
        output, finished = mx_linear_contract(bf_in, bf_weight, mx_specs["a_elem_format"],
                                              mx_specs["w_elem_format"], mx_specs,
                                              mx_specs["round_mx_output"],
                                              out_round=mx_specs["round_output"], bias=bf_bias,
                                              packed_w=packed_weight)
        if not finished:
            output = quantize_elemwise_op(output, mx_specs=mx_specs, round=mx_specs["round_output"])
            if bias is not None:
                output = quantize_elemwise_op(output + bf_bias, mx_specs=mx_specs,
                                              round=mx_specs["round_output"])
        ctx.mx_specs = get_backwards_mx_specs(mx_specs)
        ctx.prequantized_weights = prequantized_weights
        ctx.name = name
        return output

    @staticmethod
    def backward(ctx, grad_output):
        assert ctx.prequantized_weights == False, "Cannot use prequantized weights when training!"
        input, weight = ctx.saved_tensors
        specs = ctx.mx_specs
        out_dim, in_dim = weight.shape
        grad_output = quantize_elemwise_op(grad_output, mx_specs=specs,
                                           round=specs["round_grad_input"])

        # grad_weight = grad_output^T x input, contracted over the example axis; both operands share
        # exponents along axis -2 of the N-D tensors (mx/linear.py:124-143).  When that axis is a whole
        # number of blocks, no block straddles two batch entries and the tensors can be flattened to
        # 2-D first (one GEMM over all examples); block_size 0 means one block per batch entry
        block = specs["block_size"]
        if input.dim() == 2 or (input.dim() > 2 and block > 0 and input.shape[-2] % block == 0):
            grad_weight = mx_grad_contract(
                grad_output.reshape(-1, out_dim), specs["a_elem_format_bp_ex"],
                specs["round_mx_grad_output_grad_weight"], True,
                input.reshape(-1, in_dim), specs["a_elem_format_bp"],
                specs["round_mx_input_grad_weight"], True, specs)
        else:
            q_in = quantize_mx_op(input, specs, elem_format=specs["a_elem_format_bp"], axes=[-2],
                                  round=specs["round_mx_input_grad_weight"])
            q_go = quantize_mx_op(grad_output, specs, elem_format=specs["a_elem_format_bp_ex"],
                                  axes=[-2], round=specs["round_mx_grad_output_grad_weight"])
            grad_weight = torch_matmul(q_go.reshape(-1, out_dim).transpose(0, 1),
                                       q_in.reshape(-1, in_dim))
        grad_weight = quantize_elemwise_op(grad_weight, mx_specs=specs,
                                           round=specs["round_grad_weight"])

        # grad_input = grad_output x weight, contracted over the output-feature axis
        grad_input = mx_grad_contract(
            grad_output, specs["a_elem_format_bp_os"], specs["round_mx_grad_output_grad_input"], False,
            weight, specs["w_elem_format_bp"], specs["round_mx_weight_grad_input"], True, specs)
        grad_input = quantize_elemwise_op(grad_input, mx_specs=specs, round=specs["round_grad_input"])

        grad_bias = None
        if ctx.has_bias:
            grad_bias = quantize_elemwise_op(grad_output.reshape(-1, out_dim).sum(0),
                                             mx_specs=specs, round=specs["round_grad_weight"])
        return (grad_input, grad_weight, grad_bias, None, None, None, None)


def linear(input, weight, bias=None, mx_specs=None, prequantized_weights=False, name=None,
           packed_weight=None):
    """mx/linear.py:203-213.  packed_weight (not in the reference): the weight's MX codes and scales as
    Linear.prequantize_weights keeps them; the forward pass then skips the weight's quantization."""
    mx_assert_test(mx_specs)
    if mx_specs is None:
        return f_linear(input, weight, bias=bias)
    mx_specs = apply_mx_specs(mx_specs)
    return LinearFunction.apply(input, weight, bias, mx_specs, prequantized_weights, name, packed_weight)


class Linear(torch.nn.Linear):
    def __init__(self, in_features, out_features, bias=True, mx_specs=None, name=None):
        mx_assert_test(mx_specs)
        self.mx_none = mx_specs is None
        self.name = name
        self.prequantized_weights = False
        self._packed_weight = None
        self._keep_dense = True
        self.mx_specs = apply_mx_specs(mx_specs)
        super().__init__(in_features, out_features, bias)

    def apply_mx_specs(self, mx_specs):
        mx_assert_test(mx_specs)
        self.mx_none = mx_specs is None
        self.mx_specs = apply_mx_specs(mx_specs)

    def append_name(self, postfix):
        self.name += postfix

    def prequantize_weights(self, keep_dense=True):
        """Store weight and bias as bfloat16 once, for inference (mx/linear.py:246-274).  On a GPU the
        weight's MX form -- element codes + one E8M0 scale byte per block of 32, what the forward
        pass would otherwise rebuild from the bf16 weight on every call -- is built once as well, at
        the first forward pass (the layer may still move between devices until then), and the fused
        GEMM reads it directly: 1 + 1/32 bytes per weight (1/2 + 1/32 when both formats are fp4)
        against 2.  keep_dense=False also drops the bf16 weight once its codes exist (weight.data
        becomes an empty tensor): the layer then holds a half to a quarter of the bytes and serves
        bf16 GPU inputs through the fused GEMM only (anything else raises).  The codes and scales
        then are buffers of the module (weight_codes, weight_scales, weight_code_kind): they move
        with .to() / .cuda() and are part of state_dict(), and a fresh layer loads such a state.
        The cached form of a kept weight follows the weight's version counter and device; after
        changing weight.data in place (which bumps no counter) call prequantize_weights() again."""
        if self._dense_dropped():
            raise RuntimeError("prequantize_weights: the dense weight of this layer has been dropped already")
        self._keep_dense = keep_dense
        self._packed_weight = None
        if self.mx_none:
            return
        assert self.mx_specs["round"] == 'even', \
            "Bfloat round should be 'even' for prequantizing weights."
        assert torch.cuda.is_bf16_supported(), "Current device does not support bfloat16"
        assert self.mx_specs['bfloat_subnorms'] == True, \
            "Bfloat_subnorms should be set to True for prequantizing weights."
        assert self.mx_specs["bfloat"] == 16, "Only Bfloat16 is supported for prequantizing weights."
        with torch.no_grad():
            self.weight.data = quantize_elemwise_op(
                self.weight.data, mx_specs=self.mx_specs,
                round=self.mx_specs["round_weight"]).to(torch.bfloat16)
            if self.bias is not None:
                self.bias.data = quantize_elemwise_op(
                    self.bias.data, mx_specs=self.mx_specs,
                    round=self.mx_specs["round_weight"]).to(torch.bfloat16)
        self.prequantized_weights = True

    def _dense_dropped(self):
        return getattr(self, "weight_codes", None) is not None

    def _packed(self, inputs):
        """The MX form of the prequantized weight for this input, or None."""
        from . import fused
        from .gemm import fused_enabled
        if not (self.prequantized_weights and fused_enabled() and inputs.is_cuda
                and inputs.dtype == torch.bfloat16):
            return None
        if self._dense_dropped():
            if self.weight_codes.device != inputs.device:
                return None
            return (self.weight_codes, self.weight_scales, int(self.weight_code_kind))
        w = self.weight
        key = (w.data_ptr(), w._version, w.device, tuple(w.shape))
        if self._packed_weight is None or self._packed_weight[0] != key:
            if not w.is_cuda or w.numel() == 0:
                return None
            packed = fused.pack_weight(w.data, self.mx_specs["a_elem_format"], self.mx_specs["w_elem_format"],
                                       self.mx_specs, self.mx_specs["round_mx_output"])
            if packed is None:
                return None
            if not self._keep_dense:
                codes, scales, kind = packed
                self.register_buffer("weight_codes", codes)
                self.register_buffer("weight_scales", scales)
                self.register_buffer("weight_code_kind", torch.tensor(int(kind), dtype=torch.int32))
                with torch.no_grad():
                    self.weight.data = torch.empty(0, dtype=w.dtype, device=w.device)
                self._packed_weight = None
                return packed
            self._packed_weight = (key, packed)
        return self._packed_weight[1]

    def packed_weight_bytes(self):
        """Bytes of the MX form the layer holds (codes + scales), 0 before the first GPU forward pass."""
        if self._dense_dropped():
            return self.weight_codes.numel() + self.weight_scales.numel()
        if getattr(self, "_packed_weight", None) is None:
            return 0
        codes, scales, _ = self._packed_weight[1]
        return codes.numel() + scales.numel()

    def _load_from_state_dict(self, state_dict, prefix, *args, **kwargs):
        # a state saved after prequantize_weights(keep_dense=False): codes and scales instead of the weight
        codes = state_dict.get(prefix + "weight_codes")
        if codes is not None and not self._dense_dropped():
            dev = self.weight.device
            self.register_buffer("weight_codes", torch.empty_like(codes, device=dev))
            self.register_buffer("weight_scales", torch.empty_like(state_dict[prefix + "weight_scales"], device=dev))
            self.register_buffer("weight_code_kind", torch.zeros((), dtype=torch.int32))
            with torch.no_grad():
                self.weight.data = torch.empty(0, dtype=torch.bfloat16, device=dev)
                if self.bias is not None:
                    self.bias.data = self.bias.data.to(torch.bfloat16)
            self.prequantized_weights = True
            self._keep_dense = False
            self._packed_weight = None
        super()._load_from_state_dict(state_dict, prefix, *args, **kwargs)

    def forward(self, inputs):
        if self.mx_none:
            return super().forward(inputs)
        packed = None
        if self.prequantized_weights:
            assert self.training == False, "Cannot use prequantized weights when training!"
            packed = self._packed(inputs)
            if packed is None and self._dense_dropped():
                raise RuntimeError(
                    "Linear: this layer dropped its dense weight (prequantize_weights(keep_dense=False)) and holds "
                    "only MX codes on %s: it serves bfloat16 inputs on that device through the fused GEMM "
                    "(gemm.set_fused(True)), not a %s input on %s" % (self.weight_codes.device, inputs.dtype, inputs.device))
        return linear(input=inputs, weight=self.weight, bias=self.bias, mx_specs=self.mx_specs,
                      prequantized_weights=self.prequantized_weights, name=self.name, packed_weight=packed)
