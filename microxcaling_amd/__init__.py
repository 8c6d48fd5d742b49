"""MI355X-native MX / bfloat quantization with the call surface of microsoft/microxcaling.

    from microxcaling_amd.mx_ops import quantize_mx_op, _quantize_mx
    from microxcaling_amd.elemwise_ops import quantize_elemwise_op, _quantize_elemwise_core
    from microxcaling_amd import custom_extensions      # .funcs: the native entry points
"""
from .specs import (MxSpecs, get_default_mx_specs, get_backwards_mx_specs, apply_mx_specs,
                    add_mx_args, finalize_mx_specs, get_mx_specs, mx_assert_test)
from .formats import ElemFormat, RoundingMode
from .mx_ops import quantize_mx_op
from .elemwise_ops import quantize_elemwise_op
from .quantize import quantize_bfloat
from .linear import Linear, linear
from .matmul import matmul
from .bmm import bmm, bmm_softmax
from .softmax import Softmax, softmax
from .layernorm import LayerNorm, RMSNorm, layer_norm
from .activations import (sigmoid, tanh, relu, relu6, leaky_relu, silu, gelu,
                          Sigmoid, Tanh, ReLU, ReLU6, LeakyReLU, SiLU, GELU)
from .convolution import Conv1d, Conv2d, Conv3d, conv1d, conv2d, conv3d
