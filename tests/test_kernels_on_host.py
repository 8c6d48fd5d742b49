"""The HIP kernels of libmxq_gfx950.so, executed on the CPU.

Every translation unit of the GPU library -- mxq_capi.hip (quantizers, reductions), mxq_capi_gemm.hip (pack,
unpack, the 128 x 128 GEMM and the persistent 256 x 256 GEMM), mxq_capi_scores.hip (attention scores),
mxq_capi_chain.hip / mxq_capi_norm.hip (softmax, activation, vector-op and normalization kernels) -- is compiled
for the host behind tests/cpp/emu/hip/hip_runtime.h.  This file rewrites, textually, what C++ for the host cannot
express: kernel launches become calls that run the workgroups one after another with every lane a thread, and the
few inline-assembly statements become calls (copies from memory into LDS), meeting points of a wave (waits) or
nothing (register pins).  The stand-in supplies the wave-level instructions: DPP moves, shuffles, votes,
readfirstlane, v_permlane16_swap and the scaled matrix instructions v_mfma_scale_f32_32x32x64 / 16x16x128_f8f6f4
with the hardware's operand, scale and accumulator layouts.  The GPU-marked tests then run against that library
(tests/hip_on_host_plugin.py): same sources, same launch geometry and kernel selection, same ctypes signatures as
libmxq_gfx950.so, the same Python layers on top (tensors report is_cuda, so packed operands, the MFMA GEMM and
the one-launch attention scores are the paths taken).

What this cannot show is what only the hardware decides: its floating-point units (assumed IEEE, as the GPU
runs of the same tests confirmed), timing, and whether a wait placed in the source is *sufficient* (a copy into
LDS lands at once here, which is one of the orders the hardware allows; tests/cpp/gemm_addr_check.cpp replays
the others).  What it does show is that the kernels' own logic -- packing, lane exchanges, LDS layouts, operand
fragments and scales of every matrix instruction, epilogues, ragged tiles, dispatch -- computes the right
result, for every instantiation the tests reach, including those that no GPU has run yet.

By default a selection of about four minutes (see ESSENTIAL); MXQ_KERNELS_ON_HOST=all runs every GPU-marked
test that fits, which takes hours; MXQ_KERNELS_ON_HOST=none skips."""
import os
import subprocess
import sys

import pytest

from helpers import ROOT_DIR

# (files, -k expression) run by default: what has not run on a GPU yet, and one case of every kernel family
ESSENTIAL = [
    # quantizers: fp16 tensors, uncommon parameters, dither with ragged blocks (the instantiations no GPU has run)
    (["tests/test_zt_uncommon_parameters.py", "tests/test_zx_fp16_tensors.py"],
     "not every_code and not (uncommon_formats and not f16)"),
    # packed operands; the 128 x 128 GEMM; the persistent 256 x 256 GEMM on its smallest shape (128 tiles);
    # the codes-only Linear layer
    (["tests/test_gpu_fused.py", "tests/test_zw_packed_linear.py"],
     "(pack_then_unpack and nearest) or nibble_pack or gemm_propagates_nan or codes_only_layer or "
     "(scaled_mfma and fp8_e4m3-fp8_e4m3 and (128-128-128-1 or 2048-2048-512-2))"),
    # the attention-score kernel behind mx.softmax(mx.bmm(...)), with the softmax row kernel and the GEMM beside it
    # (also with the copies into LDS landing as late as the waits allow: see LATE)
    (["tests/test_zv_deferred_product_gpu.py"], "not_qualify or (shape1 and fp6_e2m3)"),
]
# with MXQ_KERNELS_ON_HOST=all: every GPU-marked test that fits.  Full-size shapes are out of reach of a few
# hundred threads on a few cores; one test checks that CPU tensors are refused; one replays a HIP graph
EVERYTHING = [
    (["tests/test_zt_uncommon_parameters.py", "tests/test_zx_fp16_tensors.py", "tests/test_gpu_parity.py",
      "tests/test_oracle_pins.py"],
     "not headline and not config1 and not config3 and not baseline and not errors_are_raised"),
    (["tests/test_zv_deferred_product_gpu.py", "tests/test_zw_packed_linear.py", "tests/test_zz_no_alloc.py",
      "tests/test_gpu_layers.py"], ""),
    (["tests/test_gpu_fused.py"],
     "not hip_graph and not thousands_of_tiles and not 4096 and not 2050 and not 1100 and not 600-520 and not 1024-"),
]


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
    def wait(m):
        count = re.search(r"vmcnt\((\d+)\)", m.group(1))
        return "emu::wait_for_copies(%s);" % (count.group(1) if count else "-1")
    text = re.sub(r'asm volatile\("(s_waitcnt[^"]*)"\s*:::\s*"memory"\);', wait, text)
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


# Copies from memory into LDS land at once by default, which shows a copy issued too early (into bytes still
# being read).  MXQ_EMU_COPIES=late carries a copy out only when a wait no longer tolerates it, which shows a wait
# that is missing or too lenient (s_waitcnt vmcnt(9) for vmcnt(8) in the attention-score kernel gives wrong
# probabilities in this mode and goes unnoticed in the other).  Groups whose kernels use such copies:
LATE = {"tests/test_zv_deferred_product_gpu.py"}


def test_gpu_tests_pass_on_the_kernels_compiled_for_the_host(host_build):
    if os.environ.get("MXQ_KERNELS_ON_HOST") == "none":
        pytest.skip("MXQ_KERNELS_ON_HOST=none")
    everything = os.environ.get("MXQ_KERNELS_ON_HOST") == "all"
    env = dict(os.environ, MXQ_HIP_ON_HOST_LIB=host_build,
               PYTHONPATH=os.path.join(ROOT_DIR, "tests") + os.pathsep + os.environ.get("PYTHONPATH", ""))
    passed = 0
    for files, select in (EVERYTHING if everything else ESSENTIAL):
        late_too = everything and "tests/test_gpu_fused.py" in files or bool(LATE & set(files))
        for mode in (("early", "late") if late_too else ("early",)):
            res = subprocess.run([sys.executable, "-m", "pytest", "-p", "hip_on_host_plugin", "-p", "no:cacheprovider",
                                  "-q", "-x", "-m", "gpu", *(["-k", select] if select else []), *files],
                                 cwd=ROOT_DIR, env=dict(env, MXQ_EMU_COPIES=mode), capture_output=True, text=True,
                                 timeout=6 * 3600)
            tail = mode + "\n" + res.stdout[-3000:] + res.stderr[-2000:]
            assert res.returncode == 0, tail
            assert " passed" in res.stdout and "failed" not in res.stdout, tail
            passed += int(res.stdout.rsplit(" passed", 1)[0].split()[-1])
    assert passed >= (1000 if everything else 30), passed
