"""The HIP kernels of the quantizer translation unit, executed on the CPU.

microxcaling_amd/csrc/mxq_capi.hip (with mxq_kernels.h: MX quantization along any axis and over several
axes, given-max, elementwise, dither, the reductions, the closed-form bf16 kernel) is compiled for the host
behind tests/cpp/emu/hip/hip_runtime.h -- kernel launches rewritten into calls that run the workgroups
one after another, the 256 lanes of a workgroup as 256 threads meeting at __syncthreads and at the DPP /
shuffle / vote exchanges of a wave -- and the GPU-marked parity tests of those kernels then run against
that library (tests/hip_on_host_plugin.py): same .hip source, same launch geometry and kernel selection,
same ctypes signatures as libmxq_gfx950.so, checked bit for bit against the oracle and the reference's
fixtures.  What this cannot show is what only the hardware decides (its IEEE arithmetic and conversions,
which the kernels assume and the GPU runs of the same tests confirm); what it does show is that the
kernels' own logic -- vector packing, lane exchanges, ragged tiles, dispatch -- is right for every
instantiation the tests reach, including those that no GPU has run yet.

By default a selection that takes about two minutes; MXQ_KERNELS_ON_HOST=all runs every GPU-marked
quantizer test that fits (about ten minutes)."""
import os
import subprocess
import sys

import pytest

from helpers import ROOT_DIR

FILES = ["tests/test_zt_uncommon_parameters.py", "tests/test_zx_fp16_tensors.py", "tests/test_gpu_parity.py",
         "tests/test_oracle_pins.py"]
# full-size shapes are out of reach of 256 threads on a few cores; one test checks that CPU tensors are refused
TOO_LARGE = "not headline and not config1 and not config3 and not baseline and not errors_are_raised"
SLOW = " and not every_code and not config2 and not reduce_reference and not several_axes and not dither_with_the_reference"


def rewrite_launches(src):
    """kernel<...><<<grid, block, lds, stream>>>(args)  ->  emu::launch(grid, block, lds, [&] { kernel<...>(args); })"""
    out, i = [], 0
    while True:
        j = src.find("<<<", i)
        if j < 0:
            out.append(src[i:])
            return "".join(out)
        k, depth = j - 1, 0                                # back over the template argument list
        assert src[k] == ">", src[j - 60:j + 10]
        while True:
            depth += {">": 1, "<": -1}.get(src[k], 0)
            if depth == 0:
                break
            k -= 1
        start = k
        while src[start - 1].isalnum() or src[start - 1] == "_":
            start -= 1
        end = src.find(">>>", j)
        grid, blockdim, lds_bytes, _ = (part.strip() for part in src[j + 3:end].rsplit(",", 3))   # ..., stream
        assert src[end + 3] == "("
        p, depth = end + 3, 0
        while True:
            depth += {"(": 1, ")": -1}.get(src[p], 0)
            if depth == 0:
                break
            p += 1
        out.append(src[i:start])
        out.append("emu::launch(%s, %s, %s, [&] { %s(%s); })" % (grid, blockdim, lds_bytes, src[start:j], src[end + 4:p]))
        i = p + 1


def rewrite_assembly(text):
    """The inline assembly of mxq_gemm.h / mxq_bmm_softmax.h in terms of the stand-in: the copies from memory into
    LDS as calls, waits as meeting points of the wave, register pins as nothing, the dynamic LDS array as a pointer
    to the stand-in's buffer."""
    import re
    text, copies = re.subn(r'asm volatile\("s_mov_b32 m0, %0\\n\\ts_nop 0\\n\\tglobal_load_lds_dword(x4)? %1, %2"\s*::\s*'
                           r'"s"\((\w+)\),\s*"v"\((\w+)\),\s*"s"\((\w+)\)\s*:\s*"memory"\);',
                           lambda m: "emu::global_load_lds(%d, %s, %s, %s);" % (16 if m.group(1) else 4, m.group(2),
                                                                                m.group(3), m.group(4)), text)
    # a wait for the wave's own copies or LDS reads: on the hardware the lanes of a wave pass it together, and the
    # kernels count on that where one lane reads LDS bytes another lane of its wave has just fetched
    text = re.sub(r'asm volatile\("s_waitcnt[^"]*"\s*:::\s*"memory"\);', "emu::wave_meet();", text)
    # ... and in the one place where lanes of a wave hand data to each other through LDS with no wait in the source
    # (the attention-score kernel stages its output rows): a meeting point between the writes and the reads
    staged = "            const bool second = t0 + 1 < ntiles;"
    if staged in text:
        assert text.count(staged) == 1
        text = text.replace(staged, "            emu::wave_meet();\n" + staged)
    text = re.sub(r'asm volatile\(""\s*:[^;]*\);', ";", text)
    text, lds = re.subn(r"extern __shared__ __attribute__\(\(aligned\(16\)\)\) unsigned char (\w+)\[\];",
                        r"unsigned char* \1 = emu::dynamic_lds();", text)
    assert "asm volatile" not in text, "inline assembly the stand-in has no counterpart for"
    return text, copies, lds


@pytest.fixture(scope="module")
def host_build(tmp_path_factory):
    """libmxq_hip_on_host.so: mxq_capi.hip (quantizers, reductions), mxq_capi_gemm.hip (pack, unpack, both GEMM
    kernels), mxq_capi_scores.hip (the attention-score kernel), mxq_capi_chain.hip and mxq_capi_norm.hip (softmax,
    activation, vector-op and normalization kernels) with their headers: every kernel of libmxq_gfx950.so, compiled
    for the host behind the stand-in runtime."""
    tmp = tmp_path_factory.mktemp("hip_on_host")
    csrc = os.path.join(ROOT_DIR, "microxcaling_amd", "csrc")
    for name, expect in (("mxq_gemm.h", (2, 1)), ("mxq_bmm_softmax.h", (0, 0))):
        with open(os.path.join(csrc, name)) as f:
            header, copies, lds = rewrite_assembly(f.read())
        assert (copies, lds) == expect, name
        with open(str(tmp / name), "w") as f:                    # found before the original on the include path
            f.write(header)
    with open(os.path.join(csrc, "mxq_capi_chain.h")) as f:       # launch macros shared by two translation units
        text = rewrite_launches(f.read())
    with open(str(tmp / "mxq_capi_chain.h"), "w") as f:
        f.write(text)
    sources, launches = [], text.count("emu::launch(")
    for unit in ("mxq_capi.hip", "mxq_capi_gemm.hip", "mxq_capi_scores.hip", "mxq_capi_chain.hip", "mxq_capi_norm.hip"):
        with open(os.path.join(csrc, unit)) as f:
            text = rewrite_launches(f.read())
        assert "<<<" not in text
        launches += text.count("emu::launch(")
        sources.append(str(tmp / (unit[:-4] + "_on_host.cpp")))
        with open(sources[-1], "w") as f:
            f.write(text)
    assert launches >= 50
    lib, emu = str(tmp / "libmxq_hip_on_host.so"), os.path.join(ROOT_DIR, "tests", "cpp", "emu")
    clang = ["/opt/rocm/lib/llvm/bin/clang++", "-std=c++20", "-fPIC", "-ffp-contract=off", "-pthread", "-msse4.1"]
    # the kernels without optimization (hundreds of instantiations: seconds instead of minutes), the arithmetic
    # of the stand-in's matrix instruction with
    subprocess.run([*clang, "-O2", "-c", os.path.join(emu, "emu_math.cpp"), "-o", str(tmp / "emu_math.o")],
                   check=True, capture_output=True, text=True, timeout=600)
    subprocess.run([*clang, "-O0", "-shared", "-I" + str(tmp), "-I" + emu, "-I" + os.path.join(ROOT_DIR, "include"),
                    "-I" + csrc, "-o", lib, *sources, str(tmp / "emu_math.o")],
                   check=True, capture_output=True, text=True, timeout=1800)
    return lib


def test_gpu_parity_tests_pass_on_the_kernels_compiled_for_the_host(host_build):
    everything = os.environ.get("MXQ_KERNELS_ON_HOST") == "all"
    env = dict(os.environ, MXQ_HIP_ON_HOST_LIB=host_build,
               PYTHONPATH=os.path.join(ROOT_DIR, "tests") + os.pathsep + os.environ.get("PYTHONPATH", ""))
    res = subprocess.run([sys.executable, "-m", "pytest", "-p", "hip_on_host_plugin", "-p", "no:cacheprovider", "-q", "-x",
                          "-m", "gpu", "-k", TOO_LARGE + ("" if everything else SLOW), *FILES],
                         cwd=ROOT_DIR, env=env, capture_output=True, text=True, timeout=3400)
    tail = res.stdout[-3000:] + res.stderr[-2000:]
    assert res.returncode == 0, tail
    assert " passed" in res.stdout and "failed" not in res.stdout, tail
    assert int(res.stdout.rsplit(" passed", 1)[0].split()[-1]) >= (190 if everything else 140), tail
