"""Writes reference_specs.json: what the reference's mx/specs.py returns for a list of spec dictionaries and
command lines -- defaults, finalize_mx_specs (dependent entries), get_backwards_mx_specs, apply_mx_specs,
add_mx_args + get_mx_specs.  Run once where the reference checkout exists:
``python tests/golden/gen_reference_specs.py /root/reference``.  Only inputs and returned dictionaries are
stored."""
import argparse
import json
import os
import sys

HERE = os.path.dirname(os.path.abspath(__file__))

SPEC_DICTS = [
    {},
    {"w_elem_format": "fp8_e4m3", "a_elem_format": "fp8_e4m3", "block_size": 32},
    {"w_elem_format": "fp4_e2m1", "a_elem_format": "fp6_e2m3", "block_size": 32, "bfloat": 16},
    {"a_elem_format": "int8", "a_elem_format_bp_os": "fp8_e5m2", "block_size": 64, "scale_bits": 8},
    {"bfloat": 16},
    {"fp": 16, "round": "even"},
    {"bfloat": 16, "round": "floor", "round_output": "nearest", "round_mx_output": "even"},
    {"w_elem_format": "fp8_e5m2", "quantize_backprop": False, "bfloat_subnorms": False},
    {"w_elem_format": "fp6_e3m2", "a_elem_format": "fp6_e3m2", "w_elem_format_bp": "fp8_e4m3", "block_size": 32,
     "shared_exp_method": "max", "mx_flush_fp32_subnorms": True, "softmax_exp2": True, "vec_use_exp2": True,
     "vec_use_recip": True},
    {"a_elem_format": "fp8_e4m3", "round_weight": "even", "round_grad_input": "floor", "round_grad_weight": "even",
     "round_mx_input_grad_input": "floor", "round_mx_weight_grad_input": "even",
     "round_mx_grad_output_grad_input": "floor", "round_mx_input_grad_weight": "even",
     "round_mx_grad_output_grad_weight": "floor"},
]

COMMAND_LINES = [
    [],
    ["--w_elem_format", "fp8_e4m3", "--a_elem_format", "fp8_e4m3", "--block_size", "32"],
    ["--bfloat", "16", "--round", "even", "--no_quantize_backprop"],
    ["--a_elem_format", "fp4_e2m1", "--scale_bits", "8", "--block_size", "32", "--softmax_exp2", "--vec_use_recip",
     "--no_bfloat_subnorms"],
    ["--skip_early_exit"],
    ["--fp", "16", "--mx_flush_fp32_subnorms", "--round_mx_output", "floor"],
]


def plain(d):
    return None if d is None else {k: d[k] for k in sorted(d.keys())}


def main(ref_root):
    sys.path.insert(0, ref_root)
    from mx import specs as S
    out = {"defaults": plain(S.get_default_mx_specs()), "finalize": [], "finalize_no_early_exit": [],
           "backwards": [], "apply": [], "command_lines": [], "argparse_defaults": None}
    for d in SPEC_DICTS:
        out["finalize"].append({"in": d, "out": plain(S.finalize_mx_specs(dict(d)))})
        f = S.finalize_mx_specs(dict(d), early_exit=False)
        out["finalize_no_early_exit"].append({"in": d, "out": plain(f)})
        out["backwards"].append({"in": d, "out": plain(S.get_backwards_mx_specs(f))})
        out["apply"].append({"in": d, "out": plain(S.apply_mx_specs(dict(d)))})
    parser = S.add_mx_args(argparse.ArgumentParser())
    out["argparse_defaults"] = {k: v for k, v in sorted(vars(parser.parse_args([])).items())}
    for argv in COMMAND_LINES:
        args = S.add_mx_args(argparse.ArgumentParser()).parse_args(argv)
        out["command_lines"].append({"in": argv, "out": plain(S.get_mx_specs(args))})
    # mx/formats.py: every element format's parameters, by name and through the enum; the enums' members
    from mx import formats as F
    names = sorted(F.ElemFormat.__members__)
    out["formats"] = {n: list(F._get_format_params(n)) for n in names}
    out["formats_by_enum"] = {n: list(F._get_format_params(F.ElemFormat[n])) for n in names}
    out["elem_format_values"] = {n: F.ElemFormat[n].value for n in names}
    out["rounding_modes"] = {n: int(F.RoundingMode[n]) for n in F.RoundingMode.__members__}
    out["rounding_mode_strings"] = list(F.RoundingMode.string_enums())
    out["min_norm"] = {str(e): F._get_min_norm(e) for e in range(0, 9)}
    out["max_norm"] = {"%d,%d" % (e, m): F._get_max_norm(e, m) for e in (5, 8) for m in (3, 4, 5, 9, 12)}
    with open(os.path.join(HERE, "reference_specs.json"), "w") as f:
        json.dump(out, f, indent=1, sort_keys=True)
    print("wrote reference_specs.json: %d spec dictionaries, %d command lines" % (len(SPEC_DICTS), len(COMMAND_LINES)))


if __name__ == "__main__":
    main(sys.argv[1] if len(sys.argv) > 1 else "/root/reference")
