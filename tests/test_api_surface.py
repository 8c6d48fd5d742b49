"""The host-side mirror of the reference's interface: formats, specs, spec-driven entry points."""
import argparse

import pytest
import torch

from helpers import assert_bits_equal
from oracle import mx_oracle as O
import microxcaling_amd as mx
from microxcaling_amd.formats import ElemFormat, RoundingMode, _get_format_params
from microxcaling_amd.specs import (MxSpecs, add_mx_args, apply_mx_specs, finalize_mx_specs,
                                    get_backwards_mx_specs, get_default_mx_specs, get_mx_specs)
from microxcaling_amd.mx_ops import quantize_mx_op
from microxcaling_amd.elemwise_ops import quantize_elemwise_op, _quantize_bfloat, _quantize_fp


def test_format_params_match_closed_forms():
    """mx/tests/test_formats.py:12-95."""
    for name in ("float16", "fp16", "bfloat16", "bf16", "fp8_e5m2", "fp8_e4m3", "fp6_e3m2",
                 "fp6_e2m3", "fp4_e2m1", "fp4", "int8", "int4", "int2"):
        assert _get_format_params(name) == O.format_params(name), name
    assert _get_format_params(ElemFormat.fp8_e4m3)[3] == 448.0
    assert [int(m) for m in RoundingMode] == [0, 1, 2]
    assert RoundingMode.string_enums() == ["nearest", "floor", "even"]
    assert ElemFormat.from_str("FP4") is ElemFormat.fp4_e2m1
    with pytest.raises(Exception):
        ElemFormat.from_str("fp5")


def test_specs_defaults_and_dependencies():
    d = get_default_mx_specs()
    assert d["scale_bits"] == 0 and d["round"] == "nearest" and d["custom_cuda"] is False
    assert d["bfloat_subnorms"] is True and d["shared_exp_method"] == "max"
    assert finalize_mx_specs({}) is None
    s = finalize_mx_specs({"w_elem_format": "fp8_e4m3", "a_elem_format": "fp6_e2m3",
                           "a_elem_format_bp_os": "fp4_e2m1", "round": "even", "block_size": 32})
    assert s["w_elem_format_bp"] == "fp8_e4m3" and s["a_elem_format_bp_ex"] == "fp6_e2m3"
    assert s["a_elem_format_bp_os"] == "fp4_e2m1"
    assert s["round_mx_output"] == "even" and s["round_mx_input_grad_input"] == "even"
    with pytest.raises(KeyError):
        apply_mx_specs({"no_such_key": 1})
    with pytest.raises(AssertionError):
        MxSpecs({"no_such_key": 1})
    b = get_backwards_mx_specs(MxSpecs({"quantize_backprop": False, "bfloat": 16, "block_size": 32}))
    assert b["bfloat"] == 0 and b["block_size"] == 0


def test_specs_argparse_round_trip():
    """mx/tests/test_finalize_mxfp.py:17-43 and the self-test at mx/specs.py:366-388."""
    p = add_mx_args(argparse.ArgumentParser())
    assert get_mx_specs(p.parse_args([])) is None
    s = get_mx_specs(p.parse_args(["--bfloat", "16", "--no_quantize_backprop", "--custom_cuda"]
                                  if torch.cuda.is_available() else ["--bfloat", "16", "--no_quantize_backprop"]))
    assert s["bfloat"] == 16 and s["quantize_backprop"] is False
    for k, v in get_default_mx_specs().items():
        if k not in ("bfloat", "quantize_backprop", "custom_cuda"):
            assert s[k] == v, k
    s = get_mx_specs(p.parse_args(["--w_elem_format", "fp6_e3m2", "--block_size", "32", "--skip_early_exit"]))
    assert s["w_elem_format_bp"] == "fp6_e3m2" and s["block_size"] == 32


def test_spec_driven_ops_on_cpu_tensors():
    g = torch.Generator().manual_seed(1)
    x = torch.randn(8, 64, generator=g)
    specs = finalize_mx_specs({"a_elem_format": "fp8_e4m3", "block_size": 32, "bfloat": 16})
    y = quantize_mx_op(x, specs, elem_format=specs["a_elem_format"], axes=[-1], round="floor")
    assert_bits_equal(y, O.quantize_mx(x, 8, "fp8_e4m3", axes=[-1], block_size=32, round="floor"))
    assert quantize_mx_op(x, specs, elem_format=None) is x
    y = quantize_elemwise_op(x, specs)
    assert_bits_equal(y, O.quantize_bfloat(x, 16))
    specs["round"] = "even"
    assert quantize_elemwise_op(x, specs).dtype == torch.bfloat16          # torch cast shortcut
    assert quantize_elemwise_op(x, None) is x
    bad = get_default_mx_specs()
    bad["bfloat"], bad["fp"] = 16, 16
    with pytest.raises(ValueError):
        quantize_elemwise_op(x, bad)
    assert _quantize_bfloat(x, 32) is x and _quantize_fp(x) is x
    assert_bits_equal(_quantize_fp(x, exp_bits=5, mantissa_bits=10, round="even"), x.half().float())


def test_sparse_coo_values_are_quantized():
    from microxcaling_amd.elemwise_ops import _quantize_elemwise_core
    x = torch.tensor([[0.0, 1.2345], [3.21, 0.0]]).to_sparse()
    y = _quantize_elemwise_core(x, 9, 8, 2 ** 127 * 255 / 128, round="even")
    assert y.is_sparse
    assert_bits_equal(y.to_dense(), x.to_dense().to(torch.bfloat16).float())


def test_fp16_tensors_in_both_exponent_modes():
    """fp16 tensors.  Default ('torch') mode: every op rounded to fp16, like the reference's pure path
    (mx/mx_ops.py:265-292, mx/elemwise_ops.py:127-163) -- compared with the oracle here and with the
    reference's own outputs in test_oracle_pins.py.  'exact' mode: the semantics of the reference's CUDA
    kernels (mx/cpp/mx.cuh:72,88): widen to fp32, quantize with bit-field exponents, round back."""
    from microxcaling_amd import custom_extensions as ce
    from microxcaling_amd.elemwise_ops import _quantize_elemwise_core
    from microxcaling_amd.mx_ops import _quantize_mx
    from oracle import mx_oracle as O
    g = torch.Generator().manual_seed(1)
    x = (torch.randn(8, 64, generator=g) * 3).half()
    for rnd in ("nearest", "floor", "even"):
        assert_bits_equal(_quantize_mx(x, 8, "fp8_e4m3", axes=[-1], block_size=32, round=rnd),
                          O.quantize_mx(x, 8, "fp8_e4m3", axes=[-1], block_size=32, round=rnd), "mx " + rnd)
        assert_bits_equal(_quantize_elemwise_core(x, 9, 8, 2 ** 127 * 255 / 128, round=rnd),
                          O.quantize_elemwise_core(x, 9, 8, 2 ** 127 * 255 / 128, round=rnd), "elementwise " + rnd)
    # the clamp of the saturating branch needs its bound in fp16: the reference raises, and so does this
    with pytest.raises(RuntimeError, match="float16"):
        _quantize_elemwise_core(x, 9, 8, 2 ** 127 * 255 / 128, saturate_normals=True)
    ce.set_exponent_mode("exact")
    try:
        for rnd in ("nearest", "floor", "even"):
            y = _quantize_mx(x, 8, "fp6_e2m3", axes=[-1], block_size=32, round=rnd)
            wide = _quantize_mx(x.float(), 8, "fp6_e2m3", axes=[-1], block_size=32, round=rnd)
            assert y.dtype == torch.float16
            assert_bits_equal(y, wide.half(), "mx " + rnd)
            y = _quantize_elemwise_core(x, 5, 4, 448.0, round=rnd, saturate_normals=True)
            wide = _quantize_elemwise_core(x.float(), 5, 4, 448.0, round=rnd, saturate_normals=True)
            assert_bits_equal(y, wide.half(), "elementwise " + rnd)
    finally:
        ce.set_exponent_mode("torch")


def test_specs_module_against_the_reference_fixture():
    """Defaults, finalize_mx_specs (dependent entries, early exit), get_backwards_mx_specs, apply_mx_specs and
    add_mx_args + get_mx_specs return what the reference's mx/specs.py returned for the same dictionaries and
    command lines (tests/golden/gen_reference_specs.py wrote them down)."""
    import argparse
    import json
    import os
    from helpers import ROOT_DIR
    from microxcaling_amd import specs as S
    ref = json.load(open(os.path.join(ROOT_DIR, "tests", "golden", "reference_specs.json")))
    plain = lambda d: None if d is None else {k: d[k] for k in sorted(d.keys())}
    assert plain(S.get_default_mx_specs()) == ref["defaults"]
    for case in ref["finalize"]:
        assert plain(S.finalize_mx_specs(dict(case["in"]))) == case["out"], case["in"]
    for case, back, app in zip(ref["finalize_no_early_exit"], ref["backwards"], ref["apply"]):
        f = S.finalize_mx_specs(dict(case["in"]), early_exit=False)
        assert plain(f) == case["out"], case["in"]
        assert plain(S.get_backwards_mx_specs(f)) == back["out"], case["in"]
        assert plain(S.apply_mx_specs(dict(app["in"]))) == app["out"], app["in"]
    parser = S.add_mx_args(argparse.ArgumentParser())
    assert {k: v for k, v in sorted(vars(parser.parse_args([])).items())} == ref["argparse_defaults"]
    for case in ref["command_lines"]:
        args = S.add_mx_args(argparse.ArgumentParser()).parse_args(case["in"])
        assert plain(S.get_mx_specs(args)) == case["out"], case["in"]
    with pytest.raises(KeyError, match="Unknown key"):
        S.apply_mx_specs({"no_such_spec": 1})


def test_formats_module_against_the_reference_fixture():
    """mx/formats.py: _get_format_params for every member of ElemFormat (by name and through the enum), the
    enums' members and values, _get_min_norm / _get_max_norm."""
    import json
    import os
    from helpers import ROOT_DIR
    from microxcaling_amd import formats as F
    ref = json.load(open(os.path.join(ROOT_DIR, "tests", "golden", "reference_specs.json")))
    assert sorted(F.ElemFormat.__members__) == sorted(ref["formats"])
    for n, want in ref["formats"].items():
        assert list(F._get_format_params(n)) == want, n
        assert list(F._get_format_params(F.ElemFormat[n])) == ref["formats_by_enum"][n], n
        assert F.ElemFormat[n].value == ref["elem_format_values"][n]
        assert F.ElemFormat.from_str(n.upper()) is F.ElemFormat[n]
    assert {n: int(F.RoundingMode[n]) for n in F.RoundingMode.__members__} == ref["rounding_modes"]
    assert list(F.RoundingMode.string_enums()) == ref["rounding_mode_strings"]
    for e, want in ref["min_norm"].items():
        assert F._get_min_norm(int(e)) == want
    for em, want in ref["max_norm"].items():
        e, m = (int(v) for v in em.split(","))
        assert F._get_max_norm(e, m) == want
    with pytest.raises(Exception, match="Undefined elem format"):
        F.ElemFormat.from_str("fp7")


def _none_cases():
    import torch.nn as nn
    import torch.nn.functional as F
    import microxcaling_amd as mx
    return [
        ("sigmoid", torch.sigmoid, mx.sigmoid, {}), ("tanh", torch.tanh, mx.tanh, {}), ("relu", F.relu, mx.relu, {}),
        ("relu6", F.relu6, mx.relu6, {}), ("leaky_relu", F.leaky_relu, mx.leaky_relu, {"negative_slope": 0.4}),
        ("silu", F.silu, mx.silu, {}), ("softmax", F.softmax, mx.softmax, {"dim": -1}),
        ("Sigmoid", nn.Sigmoid, mx.Sigmoid, {}), ("Tanh", nn.Tanh, mx.Tanh, {}), ("ReLU", nn.ReLU, mx.ReLU, {}),
        ("ReLU6", nn.ReLU6, mx.ReLU6, {}), ("SiLU", nn.SiLU, mx.SiLU, {}), ("Softmax", nn.Softmax, mx.Softmax, {"dim": -1}),
    ]


@pytest.mark.parametrize("case", range(13))
def test_without_specs_every_layer_is_the_torch_layer(case):
    """mx_specs=None: outputs and input gradients equal torch's own, bit for bit (the reference's
    mx/tests/test_mxfp_none.py:30-141, for the functions and modules this package carries)."""
    import torch.nn as nn
    name, f1, f2, kwargs = _none_cases()[case]
    g = torch.Generator().manual_seed(0xBEEF + case)
    x = torch.randn(4, 16, generator=g)
    x1, x2 = x.clone().requires_grad_(True), x.clone().requires_grad_(True)
    if isinstance(f1, type) and issubclass(f1, nn.Module):
        q1, q2 = f1(**kwargs)(x1), f2(mx_specs=None, **kwargs)(x2)
    else:
        q1, q2 = f1(x1, **kwargs), f2(x2, mx_specs=None, **kwargs)
    (q1 ** 2).mean().sqrt().backward()
    (q2 ** 2).mean().sqrt().backward()
    assert torch.equal(q1, q2), name
    assert torch.equal(x1.grad, x2.grad), name


def test_without_specs_the_matmul_layers_are_torch_layers():
    """The same for linear / Linear, matmul (with and without bias), bmm, layer_norm / LayerNorm and the
    convolutions."""
    import torch.nn as nn
    import torch.nn.functional as F
    import microxcaling_amd as mx
    g = torch.Generator().manual_seed(0xABCD)
    x, w, b = torch.randn(3, 8, 16, generator=g), torch.randn(12, 16, generator=g), torch.randn(12, generator=g)
    assert torch.equal(mx.linear(x, w, b, mx_specs=None), F.linear(x, w, b))
    assert torch.equal(mx.matmul(x, w.t(), mx_specs=None), torch.matmul(x, w.t()))
    assert torch.equal(mx.matmul(x[0], w.t(), bias=b, mx_specs=None), torch.addmm(b, x[0], w.t()))
    y = torch.randn(3, 16, 5, generator=g)
    assert torch.equal(mx.bmm(x, y, mx_specs=None), torch.bmm(x, y))
    torch.manual_seed(3)
    l1 = nn.Linear(16, 12)
    torch.manual_seed(3)
    l2 = mx.Linear(16, 12, mx_specs=None)
    assert torch.equal(l1(x), l2(x))
    lw, lb = torch.randn(16, generator=g), torch.randn(16, generator=g)
    assert torch.equal(mx.layer_norm(x, (16,), lw, lb, 1e-5, mx_specs=None), F.layer_norm(x, (16,), lw, lb, 1e-5))
    n1, n2 = nn.LayerNorm(16, eps=1e-12), mx.LayerNorm(16, mx_specs=None)    # the reference's default eps
    assert n2.eps == 1e-12
    assert torch.equal(n1(x), n2(x))
    cx, cw = torch.randn(2, 4, 9, 9, generator=g), torch.randn(6, 4, 3, 3, generator=g)
    assert torch.equal(mx.conv2d(cx, cw, None, 1, 1, 1, 1, mx_specs=None), F.conv2d(cx, cw, None, 1, 1, 1, 1))
    torch.manual_seed(5)
    c1 = nn.Conv2d(4, 6, 3, padding=1)
    torch.manual_seed(5)
    c2 = mx.Conv2d(4, 6, 3, padding=1, mx_specs=None)
    assert torch.equal(c1(cx), c2(cx))


def test_bench_refuses_more_than_one_gpu_and_needs_one():
    """bench.py measures one GPU: --gpus above 1 exits with a message that says so; without a GPU the default
    run fails loudly instead of timing anything on the CPU."""
    import os
    import subprocess
    import sys
    from helpers import ROOT_DIR
    bench = os.path.join(ROOT_DIR, "bench.py")
    res = subprocess.run([sys.executable, bench, "--gpus", "2"], capture_output=True, text=True, timeout=120)
    assert res.returncode != 0 and "one GPU" in (res.stdout + res.stderr)
    if not torch.cuda.is_available():
        res = subprocess.run([sys.executable, bench, "--steps", "1", "--warmup", "0", "--no-cpu-baseline"],
                             capture_output=True, text=True, timeout=300)
        assert res.returncode != 0
        assert '"metric"' not in res.stdout


def test_bench_reports_carry_the_contract_fields():
    """Everything of bench.py that needs no GPU: the two default workloads build, their CPU legs run on a
    sample, and the report functions turn timings into the JSON line of the contract (metric, value, unit,
    config.workload, roofline with bound / achieved / peak / frac / traffic, cpu_baseline)."""
    import importlib.util
    import json
    import os
    from helpers import ROOT_DIR
    spec = importlib.util.spec_from_file_location("bench_under_test", os.path.join(ROOT_DIR, "bench.py"))
    bench = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(bench)

    with open(os.path.join(ROOT_DIR, "profiles", "traffic.json")) as f:
        names = [k for k, v in json.load(f).items() if isinstance(v, dict)]
    assert bench.HEADLINE in names and bench.SECONDARY in names and "mx_bmm_softmax" in names
    for name in names:
        measured, note = bench.measured_traffic(name)
        assert note["summary"].startswith("profiles/") and os.path.exists(os.path.join(ROOT_DIR, note["summary"])), name
        current = note["kernel_sources_unchanged_since"] or note["kernel_code_compared_identical"]
        assert (measured == note["last_measured_bytes"]) if current else measured is None

    wl = bench.make_workload(bench.HEADLINE)
    assert wl["bytes"] == 8192 * 8192 * 8 and wl["x"].shape == (8192, 8192)
    assert wl["cpu"](wl["x"][:64, :64].contiguous()).shape == (64, 64)
    line = bench.bytes_report(bench.HEADLINE, wl, 200, 50, 0.0831, 0.0807, False)
    line["cpu_baseline"] = {"value": 1.0, "unit": "GB/s", "cores": 1, "kind": "port", "sample": "-"}
    sec_wl = bench.make_workload(bench.SECONDARY)
    assert sec_wl["flops"] == 2 * 16384 * 14336 * 4096
    sec_wl["cpu_rows"] = 64                                     # a smaller sample than the bench run takes
    sec = bench.flops_report(bench.SECONDARY, sec_wl, 200, 50, 0.95, 0.94, 0.85, True)
    for rep, unit, bound in ((line, "GB/s", "hbm"), (sec, "TFLOP/s", "mfma")):
        rep = json.loads(json.dumps(rep))
        assert rep["metric"] == bench.METRIC and rep["unit"] == unit and rep["n_gpus"] == 1
        assert rep["higher_is_better"] is True and rep["vs_baseline"] is None and rep["data"] == "synthetic"
        assert "workload" in rep["config"] and "model" not in rep["config"]
        roof = rep["roofline"]
        assert roof["bound"] == bound and roof["unit"] == unit and "traffic" in roof
        assert abs(roof["frac"] - roof["achieved"] / roof["peak"]) < 1e-3
        assert set(rep["cpu_baseline"]) >= {"value", "unit", "cores", "kind", "sample"}
    assert abs(line["roofline"]["achieved"] - 536870912 / 0.0807e-3 / 1e9) < 1.0
    assert abs(sec["roofline"]["achieved"] - 1924145348608 / 0.85e-3 / 1e12) < 0.1 and sec["cpu_baseline"]["value"] > 0


def test_the_reference_side_stub_of_the_integration_notes():
    """The ctypes binding a maintainer of the reference would drop in for mx/custom_extensions.py is real
    code: it loads both libraries, offers the seven names of mx/cpp/funcs.cpp:234-242, and its CPU
    functions return what the reference's pure path returns (here: the oracle)."""
    from oracle import mx_oracle as O
    from helpers import integration_stub
    stub = integration_stub()
    assert sorted(vars(stub.funcs)) == sorted([
        "quantize_mx_func_cpp", "quantize_elemwise_func_cpp", "quantize_mx_func_cuda", "quantize_mx_by_tile_func_cuda",
        "quantize_elemwise_func_cuda", "reduce_sum_inner_dim", "reduce_max_inner_dim"])
    g = torch.Generator().manual_seed(4)
    for dtype in (torch.float32, torch.bfloat16, torch.float16):
        x = (torch.randn(6, 96, generator=g) * 4).to(dtype)
        blocks = x.view(6, 3, 32)
        mx = blocks.abs().max(dim=2, keepdim=True).values
        got = stub.funcs.quantize_mx_func_cpp(blocks, 8, 4, 5, 448.0, mx, 2, False, 0).view(6, 96)
        assert_bits_equal(got, O.quantize_mx(x, 8, "fp8_e4m3", axes=[-1], block_size=32), "mx %s" % dtype)
        got = stub.funcs.quantize_elemwise_func_cpp(x, 9, 8, 2 ** 127 * 255 / 128, 2, False, True)
        assert_bits_equal(got, O.quantize_elemwise_core(x, 9, 8, 2 ** 127 * 255 / 128, round="even"), "elem %s" % dtype)
    with pytest.raises(RuntimeError, match="scale_bits"):
        stub.funcs.quantize_mx_func_cpp(torch.zeros(1, 32), 0, 4, 5, 448.0, torch.zeros(1, 1), 1, False)


@pytest.mark.parametrize("name", ["sigmoid", "tanh", "relu", "leaky_relu", "silu", "gelu", "softmax", "linear", "matmul",
                                  "bmm", "conv1d", "conv2d", "conv3d"])
def test_finite_differences_without_mx_specs(name):
    """mx/tests/test_gradcheck.py:25-89: with mx_specs None every function is torch's own and passes
    torch.autograd.gradcheck in float64 (a wrapper that dropped or reordered an argument would not)."""
    import microxcaling_amd as mx
    fn = getattr(mx, name)
    g = torch.Generator().manual_seed(0xBEEF)
    r = lambda *s: torch.randn(*s, dtype=torch.float64, generator=g).requires_grad_(True)
    if name in ("linear", "matmul"):
        args = (r(3, 8, 8), r(8, 8))
    elif name == "bmm":
        args = (r(3, 8, 8), r(3, 8, 8))
    elif name.startswith("conv"):
        nd = int(name[4])
        args = (r(2, 8, *([3] * nd)), r(2, 8, *([1] * nd)))
    elif name == "softmax":
        args = (r(64),)
        fn = lambda x: mx.softmax(x, dim=-1)
    else:
        args = (r(64),)
    assert torch.autograd.gradcheck(fn, args)


def test_the_written_notes_name_things_that_exist():
    """Every test, source file, profile summary, kernel and C symbol that the Markdown notes at the repository
    root mention in code quotes exists in the tree (notes drift when code is renamed)."""
    import glob
    import os
    import re
    from helpers import ROOT_DIR
    tests = {os.path.basename(f): open(f).read() for f in glob.glob(os.path.join(ROOT_DIR, "tests", "*.py"))}
    sources = "\n".join(open(f).read() for f in glob.glob(os.path.join(ROOT_DIR, "microxcaling_amd", "**", "*"), recursive=True)
                        if os.path.isfile(f) and f.endswith((".py", ".h", ".hip", ".cpp")))
    sources += open(os.path.join(ROOT_DIR, "include", "mxq.h")).read()
    missing = []
    for doc in ("DESIGN", "README", "INTEGRATION"):
        text = open(os.path.join(ROOT_DIR, doc + ".md")).read()
        for path, name in re.findall(r"(tests/[\w/]+\.(?:py|cpp))(?:::([\w…]+))?", text):
            if not os.path.exists(os.path.join(ROOT_DIR, path)):
                missing.append((doc, path))
            elif name and path.endswith(".py") and ("def " + name.rstrip("…")) not in tests[os.path.basename(path)]:
                missing.append((doc, path, name))
        for path in re.findall(r"`((?:profiles|include|microxcaling_amd)/[\w/.+-]+)`", text):
            if not os.path.exists(os.path.join(ROOT_DIR, path)):
                missing.append((doc, path))
        for name in set(re.findall(r"`(\w+_kernel(?:_256p)?|mxq_\w+)`", text)):
            if name not in sources:
                missing.append((doc, name))
    assert not missing, missing
