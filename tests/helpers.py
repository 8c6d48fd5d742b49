"""Shared helpers for the test-suite: bit-pattern comparison and fixture access."""
import importlib.util
import json
import os

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
GOLDEN = os.path.join(HERE, "golden")
ROOT_DIR = os.path.dirname(HERE)


def canon_bits(t):
    """Integer bit patterns of a float tensor with every NaN mapped to the canonical quiet NaN
    (NaN payloads are not part of the parity contract; the sign of zero is)."""
    t = t.detach().cpu().contiguous()
    if t.dtype == torch.float32:
        b = t.view(torch.int32).numpy()
        return np.where(np.isnan(t.numpy()), np.int32(0x7FC00000), b)
    if t.dtype == torch.bfloat16:
        b = t.view(torch.int16).numpy()
        return np.where(np.isnan(t.float().numpy()), np.int16(0x7FC0), b)
    if t.dtype == torch.float16:
        b = t.view(torch.int16).numpy()
        return np.where(np.isnan(t.float().numpy()), np.int16(0x7E00), b)
    raise TypeError(t.dtype)


def assert_bits_equal(got, want, what=""):
    g, w = canon_bits(got), canon_bits(want)
    assert g.shape == w.shape, (what, g.shape, w.shape)
    bad = np.flatnonzero(g.reshape(-1) != w.reshape(-1))
    if bad.size:
        i = int(bad[0])
        gf = got.detach().cpu().reshape(-1)[i].item()
        wf = want.detach().cpu().reshape(-1)[i].item()
        raise AssertionError("%s: %d of %d elements differ; first at flat index %d: got %r (0x%x) "
                             "want %r (0x%x)" % (what, bad.size, g.size, i, gf,
                                                 int(g.reshape(-1)[i]) & 0xFFFFFFFF, wf,
                                                 int(w.reshape(-1)[i]) & 0xFFFFFFFF))


def from_bits(a, dtype):
    t = torch.from_numpy(np.ascontiguousarray(a))
    return t.view(dtype)


_golden = None


def golden():
    """(npz arrays, json meta) written by tests/golden/gen_reference_vectors.py."""
    global _golden
    if _golden is None:
        z = np.load(os.path.join(GOLDEN, "reference_vectors.npz"))
        with open(os.path.join(GOLDEN, "reference_vectors.json")) as f:
            meta = json.load(f)
        _golden = (z, meta)
    return _golden


def golden_inputs_module():
    """The fixture generator, imported for its seeded input builders (its main() is not run)."""
    spec = importlib.util.spec_from_file_location(
        "gen_reference_vectors", os.path.join(GOLDEN, "gen_reference_vectors.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


_dither = None


def dither_golden():
    """Arrays written by tests/golden/gen_reference_dither_vectors.py, and its case tables."""
    global _dither
    if _dither is None:
        import importlib.util
        here = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
        spec = importlib.util.spec_from_file_location("gen_reference_dither_vectors",
                                                      os.path.join(here, "gen_reference_dither_vectors.py"))
        mod = importlib.util.module_from_spec(spec)
        spec.loader.exec_module(mod)
        _dither = (np.load(os.path.join(here, "reference_dither_vectors.npz")), mod)
    return _dither


def dither_cases():
    """(kind, dtype name, torch dtype, case number, seed, parameters, input tensor, expected output) for
    every stored case."""
    z, mod = dither_golden()
    for name, dtype in (("f32", torch.float32), ("bf16", torch.bfloat16), ("f16", torch.float16)):
        x = from_bits(z["x_" + name], dtype)
        for n, case in enumerate(mod.MX_CASES):
            yield "mx", name, dtype, n, 1000 + n, case, x, from_bits(z["mx_%s_%d" % (name, n)], dtype)
        for n, case in enumerate(mod.ELEM_CASES):
            yield "elem", name, dtype, n, 2000 + n, case, x, from_bits(z["elem_%s_%d" % (name, n)], dtype)


def reference_noise(kind, case, x):
    """The uniform numbers the reference hands the elements of x in a stored dither case, drawn on the CPU
    under the current torch seed: torch.rand_like of the tensor the element quantizer sees, which for MX is
    x padded to whole blocks along the block axis (mx/mx_ops.py:226-229; the padding's numbers are dropped)."""
    if kind != "mx" or case[2] <= 0 or x.shape[case[1]] % case[2] == 0:
        return torch.rand_like(x)
    _, axis, bs = case
    shape = list(x.shape)
    shape[axis] = -(-shape[axis] // bs) * bs
    return torch.rand(shape, dtype=x.dtype).narrow(axis % x.ndim, 0, x.shape[axis]).contiguous()


class PackageImpl:
    """This package's own entry points behind the call signature of the oracles, so that one test
    body can run against an oracle, against the host library (CPU tensors -> libmxq_host.so) and
    against the HIP kernels (tensors moved to the GPU and back)."""

    def __init__(self, device):
        self.device = device

    def _to(self, A):
        if self.device == "cuda":
            assert torch.cuda.is_available(), "this case needs a GPU"
        return A.to(self.device)

    def quantize_mx(self, A, scale_bits, elem_format, axes, block_size=0, round="nearest",
                    flush_fp32_subnorms=False):
        from microxcaling_amd.mx_ops import _quantize_mx
        y = _quantize_mx(self._to(A), scale_bits, elem_format, axes=axes, block_size=block_size, round=round,
                         flush_fp32_subnorms=flush_fp32_subnorms, custom_cuda=self.device == "cuda")
        return y.cpu()

    def quantize_elemwise_core(self, A, bits, exp_bits, max_norm, round="nearest", saturate_normals=False,
                               allow_denorm=True):
        from microxcaling_amd.elemwise_ops import _quantize_elemwise_core
        y = _quantize_elemwise_core(self._to(A), bits, exp_bits, max_norm, round=round,
                                    saturate_normals=saturate_normals, allow_denorm=allow_denorm,
                                    custom_cuda=self.device == "cuda")
        return y.cpu()


def integration_stub():
    """The replacement for the reference's mx/custom_extensions.py printed in INTEGRATION.md, as a module."""
    import re
    import types
    from microxcaling_amd import _lib
    text = open(os.path.join(ROOT_DIR, "INTEGRATION.md")).read()
    m = re.search(r"```python\n(# mx/custom_extensions.py  \(replacement.*?)```", text, re.S)
    assert m, "the stub is no longer in INTEGRATION.md"
    code = m.group(1).replace("/path/to/libmxq_gfx950.so", _lib.GPU_LIB_PATH).replace("/path/to/libmxq_host.so",
                                                                                     _lib.HOST_LIB_PATH)
    mod = types.ModuleType("reference_side_stub")
    exec(compile(code, "INTEGRATION.md", "exec"), mod.__dict__)
    return mod
