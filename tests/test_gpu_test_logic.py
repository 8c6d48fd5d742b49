"""The GPU-marked tests of the quantizers, run once with every cuda device mapped to the CPU
(tests/cpu_dry_run_plugin.py): their bodies then go through the host library.  This checks the tests, not
the kernels -- counts, keys, fixtures, tolerances that do not depend on the device -- so that a mistake in
a test shows up here and not in the middle of a GPU run.  Tests that call GPU-only entry points (reductions,
the *_cuda functions, packed operands, fused kernels) are left out."""
import os
import subprocess
import sys

from helpers import ROOT_DIR

QUANTIZER_FILES = ["tests/test_gpu_parity.py", "tests/test_oracle_pins.py", "tests/test_zt_uncommon_parameters.py",
                   "tests/test_zx_fp16_tensors.py", "tests/test_gpu_layers.py"]
GPU_ONLY = "not reduc and not given_max and not static_scratch"


def test_gpu_marked_quantizer_tests_run_clean_on_cpu_tensors():
    env = dict(os.environ, PYTHONPATH=os.path.join(ROOT_DIR, "tests") + os.pathsep + os.environ.get("PYTHONPATH", ""))
    res = subprocess.run([sys.executable, "-m", "pytest", "-p", "cpu_dry_run_plugin", "-p", "no:cacheprovider", "-q", "-x",
                          "-m", "gpu", "-k", GPU_ONLY, *QUANTIZER_FILES],
                         cwd=ROOT_DIR, env=env, capture_output=True, text=True, timeout=1800)
    tail = res.stdout[-3000:] + res.stderr[-2000:]
    assert res.returncode == 0, tail
    assert " passed" in res.stdout and "failed" not in res.stdout, tail
    assert int(res.stdout.rsplit(" passed", 1)[0].split()[-1]) >= 300, tail
