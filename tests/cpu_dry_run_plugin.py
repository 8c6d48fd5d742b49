"""pytest plugin (python -m pytest -p cpu_dry_run_plugin ...) that maps every "cuda" device to the CPU:
tensor.to / .cuda, module.to / .cuda, the device= argument of torch's factory functions,
torch.cuda.is_available / synchronize.  GPU-marked tests of the quantizers then run their bodies on CPU
tensors, through the host library instead of the HIP kernels.  That proves nothing about the kernels; it
finds mistakes in the tests themselves (a wrong count, a misspelt key, a fixture that is not there) before
a GPU run does.  Used by tests/test_gpu_test_logic.py only."""
import functools

import torch


def _cpu(dev):
    if isinstance(dev, str) and dev.startswith("cuda"):
        return "cpu"
    if isinstance(dev, torch.device) and dev.type == "cuda":
        return torch.device("cpu")
    return dev


def _mapped(fn):
    @functools.wraps(fn)
    def inner(*args, **kwargs):
        args = tuple(_cpu(a) if isinstance(a, (str, torch.device)) else a for a in args)
        if "device" in kwargs:
            kwargs["device"] = _cpu(kwargs["device"])
        return fn(*args, **kwargs)
    return inner


torch.cuda.is_available = lambda: True
torch.cuda.synchronize = lambda *a, **k: None
torch.Tensor.to = _mapped(torch.Tensor.to)
torch.Tensor.cuda = lambda self, *a, **k: self
torch.nn.Module.to = _mapped(torch.nn.Module.to)
torch.nn.Module.cuda = lambda self, *a, **k: self
for _name in ("ones", "zeros", "randn", "rand", "empty", "full", "linspace", "arange", "tensor", "randint", "eye",
              "as_tensor", "zeros_like", "ones_like", "empty_like", "rand_like", "randn_like", "full_like"):
    setattr(torch, _name, _mapped(getattr(torch, _name)))
