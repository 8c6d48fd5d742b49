"""The layers on CPU tensors under 40 random mx_specs in which every role (forward / each gradient,
weights / activations, every round_* key) has its own format and rounding, against what the
reference's layers returned for the same settings and inputs (tests/golden/gen_reference_spec_sweep.py;
mx/specs.py:84-116 lists the roles).  A layer that takes the wrong role's setting anywhere gives other
bits.  Bit for bit: same torch, same op order, single-threaded GEMM."""
import importlib.util
import json
import os

import numpy as np
import pytest
import torch

from helpers import GOLDEN, assert_bits_equal, from_bits

_spec = importlib.util.spec_from_file_location("gen_reference_spec_sweep",
                                               os.path.join(GOLDEN, "gen_reference_spec_sweep.py"))
GEN = importlib.util.module_from_spec(_spec)
_spec.loader.exec_module(GEN)
with open(os.path.join(GOLDEN, "reference_spec_sweep.json")) as _f:
    META = json.load(_f)
FIX = np.load(os.path.join(GOLDEN, "reference_spec_sweep.npz"))


@pytest.fixture(autouse=True)
def one_thread():
    n = torch.get_num_threads()
    torch.set_num_threads(1)
    yield
    torch.set_num_threads(n)


def test_the_sweep_settings_are_the_generators():
    assert META["cases"] == json.loads(json.dumps(GEN.spec_cases())) and len(META["cases"]) == GEN.N_CASES
    inp = GEN.inputs()
    for k, v in inp.items():
        assert_bits_equal(v, from_bits(FIX["in/" + k], torch.float32).reshape(v.shape), k)


@pytest.mark.parametrize("dname", list(GEN.DTYPES))
@pytest.mark.parametrize("case", range(GEN.N_CASES))
def test_layers_under_random_specs(case, dname):
    import microxcaling_amd as mx
    dt = GEN.DTYPES[dname]
    raw = META["cases"][case]
    got = GEN.run_case(mx, raw, GEN.inputs(), dt)
    want = {k.split("/", 2)[2]: v for k, v in META["digests"].items() if k.startswith("%d/%s/" % (case, dname))}
    assert sorted(got) == sorted(want), (sorted(set(got) ^ set(want)), raw)
    for k, v in got.items():
        if isinstance(v, str):
            assert want[k].startswith("raised:"), k          # the reference raises for this setting as well
            continue
        stored = "%d/%s/%s" % (case, dname, k)
        if stored in FIX.files:
            assert str(v.dtype).replace("torch.", "") == want[k].split(":")[0], k
            assert_bits_equal(v.detach(), from_bits(FIX[stored], v.dtype).reshape(v.shape), "%s under %s" % (k, raw))
        assert GEN.digest(v) == want[k], "%s under %s" % (k, raw)
