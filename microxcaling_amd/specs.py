"""MxSpecs: the dictionary of quantization settings every MX op reads.  Same keys, defaults,
helper names and argparse glue as the reference's mx/specs.py."""
import argparse
import collections
import json
import os
import traceback

import torch

# MX_ASSERT=True makes a missing mx_specs an error in every op (mx/specs.py:58, 351-363)
_ASSERT_MODE = os.environ.get('MX_ASSERT', 'False')

_ROUND_HELP = ""
# key -> (default, help)
_SPEC_TABLE = collections.OrderedDict([
    ("scale_bits", (0, "Bits (sign + magnitude) to use for shared exponent/scale")),
    ("w_elem_format", (None, "Weight MX elem format, one of {fp8_e5m2, fp8_e4m3, fp6_e3m2, "
                             "fp6_e2m3, fp4_e2m1, int8, int4}")),
    ("a_elem_format", (None, "Activation MX elem format. See w_elem_format")),
    ("w_elem_format_bp", (None, "Backpass weight MX elem format. See w_elem_format")),
    ("a_elem_format_bp", (None, "Backpass stashed activation MX elem format. See w_elem_format")),
    ("a_elem_format_bp_ex", (None, "Backpass act (grad) MX elem format. See w_elem_format")),
    ("a_elem_format_bp_os", (None, "Backpass act (grad) MX elem format. See w_elem_format")),
    ("mx_flush_fp32_subnorms", (False, "MX quantization flushes blocks with subnormal shared "
                                       "scale to zero")),
    ("shared_exp_method", ("max", "Shared exponent calculation method. Options: max, none")),
    ("block_size", (0, "mx shared exponent block size")),
    ("bfloat", (0, "BfloatX format (8exp + sign + mantissa). Only one of bfloat or fp can be used")),
    ("fp", (0, "fpX format (5exp + sign + mantissa). Only one of bfloat or fp can be used")),
    ("bfloat_subnorms", (True, "Bfloat/FP supports subnorms")),
    ("quantize_backprop", (True, "Enable mx/bfloat quantization on backward pass")),
    ("round", ("nearest", "Global rounding mode. Choices: nearest, floor, even")),
    ("round_m", ("nearest", "ADAM optimizer m and v rounding mode")),
    ("round_weight", ("nearest", "Weight bfloat rounding mode (W in WAGE)")),
    ("round_output", ("nearest", "Activation bfloat rounding mode (A in WAGE)")),
    ("round_grad_weight", ("nearest", "Weight update rounding mode (G in WAGE)")),
    ("round_grad_input", ("nearest", "Error gradient rounding mode (E in WAGE)")),
    ("round_mx_output", ("nearest", "Forward pass mx rounding mode")),
    ("round_mx_input_grad_input", ("nearest", _ROUND_HELP)),
    ("round_mx_weight_grad_input", ("nearest", _ROUND_HELP)),
    ("round_mx_grad_output_grad_input", ("nearest", _ROUND_HELP)),
    ("round_mx_input_grad_weight", ("nearest", _ROUND_HELP)),
    ("round_mx_grad_output_grad_weight", ("nearest", _ROUND_HELP)),
    ("softmax_exp2", (False, "Softmax uses 2^x instead of e^x")),
    ("vec_use_exp2", (False, "Use 2^x to compute e^x")),
    ("vec_use_recip", (False, "Use 1/x to compute division")),
    ("custom_cuda", (False, "Enable custom native kernels for quantization")),
])


_DEFAULTS = {k: default for k, (default, _) in _SPEC_TABLE.items()}
_HELP_STRINGS = {k: h for k, (_, h) in _SPEC_TABLE.items()}


class MxSpecs(collections.UserDict):
    """Dict of quantization parameters; unknown keys are rejected, missing keys get defaults."""

    def __init__(self, *args, **kwargs):
        super().__init__(*args, **kwargs)
        self.help_strings = _HELP_STRINGS
        given, self.data = self.data, dict(_DEFAULTS)
        self.data.update(given)
        if len(self.data) != len(_DEFAULTS):
            for k in self.data:
                assert k in _SPEC_TABLE, "unknown mx spec %r" % k

    def safe_json(self, indent=None):
        return json.dumps(self.data, indent=indent,
                          default=lambda o: f"<<non-serializable: {type(o).__qualname__}>>")

    def __str__(self):
        return self.safe_json(indent=4)


def get_default_mx_specs():
    """Specs that quantize nothing."""
    return MxSpecs()


def get_backwards_mx_specs(specs):
    """Specs for the backward pass: everything off unless quantize_backprop is set."""
    bspecs = specs.copy()
    if bspecs["quantize_backprop"] == False:
        for k in ("w_elem_format", "a_elem_format", "w_elem_format_bp", "a_elem_format_bp",
                  "a_elem_format_bp_os", "a_elem_format_bp_ex"):
            bspecs[k] = None
        bspecs["block_size"] = 0
        bspecs["bfloat"] = 0
        bspecs["fp"] = 0
    return bspecs


def apply_mx_specs(mx_specs, default_mx_specs=None):
    """Overlay the non-None entries of mx_specs on the defaults; unknown keys raise KeyError."""
    if not default_mx_specs:
        default_mx_specs = get_default_mx_specs()
    if not mx_specs:
        return default_mx_specs
    given = mx_specs.data if isinstance(mx_specs, MxSpecs) else mx_specs
    for k, v in given.items():
        if v != None:
            if k not in default_mx_specs:
                raise KeyError(f"Unknown key '{k}' passed to mx specs")
            default_mx_specs[k] = v
    return default_mx_specs


def add_mx_args(parser: argparse.ArgumentParser) -> argparse.ArgumentParser:
    """One command-line option per spec.  Non-bool options default to None (= not given); a
    default-False bool becomes --<key>, a default-True bool becomes --no_<key>."""
    group = parser.add_argument_group("mx", "MX specs")
    group.add_argument("--mx_dir", type=str, default=None, help="Path to mx library")
    for k, (default, help_str) in _SPEC_TABLE.items():
        help_str = help_str or "No help string"
        if "elem_format" in k:
            group.add_argument("--" + k, type=str, default=default, help=help_str)
        elif default is False:
            group.add_argument("--" + k, action="store_true", help=help_str)
        elif default is True:
            group.add_argument("--no_" + k, action="store_true", help=help_str)
        else:
            group.add_argument("--" + k, type=type(default), default=None, help=help_str)
    group.add_argument("--skip_early_exit", action="store_true", default=False,
                       help="Don't early exit if no quantization is specified")
    return parser


_DEPENDS = [
    ("w_elem_format_bp", "w_elem_format"), ("a_elem_format_bp", "a_elem_format"),
    ("a_elem_format_bp_os", "a_elem_format"), ("a_elem_format_bp_ex", "a_elem_format"),
    ("round_m", "round"), ("round_output", "round"), ("round_grad_weight", "round"),
    ("round_grad_input", "round"), ("round_weight", "round"), ("round_mx_output", "round"),
    ("round_mx_input_grad_input", "round_grad_input"),
    ("round_mx_weight_grad_input", "round_grad_input"),
    ("round_mx_grad_output_grad_input", "round_grad_input"),
    ("round_mx_input_grad_weight", "round_grad_input"),
    ("round_mx_grad_output_grad_weight", "round_grad_input"),
]


def finalize_mx_specs(specs, early_exit=True):
    """Fill the specs that default to another spec and return a complete MxSpecs -- or None when
    nothing is quantized (and early_exit).  Call before using a hand-written or parsed dict."""
    quantizing = any(specs.get(k, 0) for k in (
        "w_elem_format", "a_elem_format", "w_elem_format_bp", "a_elem_format_bp",
        "a_elem_format_bp_os", "a_elem_format_bp_ex", "bfloat", "fp"))
    if not quantizing and early_exit:
        return None
    if specs.get('custom_cuda'):
        assert torch.cuda.is_available(), "'custom_cuda' is only supported on CUDA devices."
    for dst, src in _DEPENDS:
        if (dst not in specs or specs[dst] is None) and src in specs:
            specs[dst] = specs[src]
    return apply_mx_specs(specs, get_default_mx_specs())


def get_mx_specs(parsed_args: argparse.Namespace):
    """MxSpecs from the namespace produced by a parser that went through add_mx_args."""
    parsed = {}
    for k, (default, _) in _SPEC_TABLE.items():
        if default is True:
            if hasattr(parsed_args, "no_" + k):
                parsed[k] = not getattr(parsed_args, "no_" + k)
        elif hasattr(parsed_args, k):
            parsed[k] = getattr(parsed_args, k)
    early_exit = not getattr(parsed_args, "skip_early_exit", False)
    return finalize_mx_specs(parsed, early_exit=early_exit)


def mx_assert_test(mx_specs):
    if _ASSERT_MODE == "True" and mx_specs is None:
        stack = traceback.extract_stack()
        op, site = stack[-2], stack[-3]
        raise ValueError("MX assert test failed!\n"
                         f"mx_specs is None in function {op.name}\n"
                         f"Called from {site.filename}, line {site.lineno}\n"
                         f"  {site.line}")
