"""The layers on CPU tensors over 45 seeded random shapes -- contraction lengths that leave a ragged
last block, inputs of rank 1 to 4, batched and plain second operands, softmax over any axis, norm
widths from 1 to 200, convolutions in one to three dimensions with stride / padding / dilation /
groups -- under three settings, against digests of what the reference's layers returned for the same
shapes and seeds (tests/golden/gen_reference_shape_sweep.py).  Outputs and every gradient, bit for bit."""
import importlib.util
import json
import os

import pytest
import torch

from helpers import GOLDEN

_spec = importlib.util.spec_from_file_location("gen_reference_shape_sweep",
                                               os.path.join(GOLDEN, "gen_reference_shape_sweep.py"))
GEN = importlib.util.module_from_spec(_spec)
_spec.loader.exec_module(GEN)
with open(os.path.join(GOLDEN, "reference_shape_sweep.json")) as _f:
    META = json.load(_f)
CASES = GEN.cases()


@pytest.fixture(autouse=True)
def one_thread():
    n = torch.get_num_threads()
    torch.set_num_threads(1)
    yield
    torch.set_num_threads(n)


def test_the_sweep_is_the_generators():
    assert META["cases"] == json.loads(json.dumps([[k, p] for k, p in CASES])) and META["settings"] == GEN.SETTINGS
    assert len(CASES) == 45 and len(META["digests"]) == 792


@pytest.mark.parametrize("ci", range(len(CASES)), ids=["%d-%s" % (i, c[0]) for i, c in enumerate(CASES)])
def test_layers_over_random_shapes(ci):
    import microxcaling_amd as mx
    kind, prm = CASES[ci]
    for si, setting in enumerate(GEN.SETTINGS):
        for dname, dt in GEN.DTYPES.items():
            if kind == "conv" and dname == "bf16":
                continue
            got = GEN.run_case(mx, kind, prm, setting, dt, 1000 * ci + si)
            prefix = "%d/%d/%s/" % (ci, si, dname)
            want = {k[len(prefix):]: v for k, v in META["digests"].items() if k.startswith(prefix)}
            assert sorted(got) == sorted(want), (kind, prm, setting, got.get("raised"))
            for k, v in got.items():
                have = v if isinstance(v, str) else GEN.digest(v)
                assert have == want[k], "%s of %s %s under setting %d, %s" % (k, kind, prm, si, dname)
