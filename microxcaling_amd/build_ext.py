"""Builds the two native libraries in-tree, next to this file.

    libmxq_gfx950.so   HIP kernels for gfx950 + the C ABI of include/mxq.h   (hipcc)
    libmxq_host.so     the same scalar arithmetic for CPU tensors            (ROCm clang++)

Usage:  python -m microxcaling_amd.build_ext
        python -m microxcaling_amd.build_ext --compare-with <commit>    (generated code, kernel by kernel)
hipcc cross-compiles, so no GPU is needed to build.
"""
import concurrent.futures
import hashlib
import os
import subprocess
import tempfile
import sys

PKG = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(PKG)
CSRC = os.path.join(PKG, "csrc")
ROCM = os.environ.get("ROCM_PATH", "/opt/rocm")

GPU_LIB = os.path.join(PKG, "libmxq_gfx950.so")
HOST_LIB = os.path.join(PKG, "libmxq_host.so")

COMMON = ["-O3", "-std=c++17", "-fPIC", "-shared", "-ffp-contract=off", "-fvisibility=hidden",
          "-I" + os.path.join(ROOT, "include"), "-I" + CSRC]


def source_digest():
    """sha256 over every file the two libraries are compiled from (names and contents).  Both builds
    compile it in (mxq_build_digest / mxq_host_build_digest), so a library can be told apart from
    one built from other sources -- the tests compare it with the tree they run in."""
    h = hashlib.sha256()
    files = [os.path.join(ROOT, "include", "mxq.h")]
    files += sorted(os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith((".h", ".hip", ".cpp")))
    for path in files:
        h.update(os.path.basename(path).encode() + b"\0")
        with open(path, "rb") as f:
            h.update(f.read())
        h.update(b"\0")
    return h.hexdigest()


def _digest_flag():
    return '-DMXQ_BUILD_DIGEST="%s"' % source_digest()


def _run(cmd, verbose):
    if verbose:
        print(" ".join(cmd), flush=True)
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    # the host pass of hipcc does not know the gfx950 target feature below and says so: harmless
    out = "\n".join(l for l in res.stdout.splitlines()
                    if "packed-fp32-ops" not in l and l.strip())
    if res.returncode != 0:
        raise RuntimeError("build failed (%d): %s\n%s" % (res.returncode, " ".join(cmd), out))
    if verbose and out:
        print(out, flush=True)


GPU_SOURCES = ["mxq_capi.hip", "mxq_capi_gemm.hip", "mxq_capi_chain.hip", "mxq_capi_norm.hip",
               "mxq_capi_scores.hip"]


def build_gpu(verbose=True):
    """Compiles the translation units side by side, then links them."""
    hipcc = os.path.join(ROCM, "bin", "hipcc")
    flags = ["--offload-arch=gfx950",
             # keep fp32 math scalar: packed fp32 instructions are not used by these kernels
             "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
             *[f for f in COMMON if f != "-shared"], _digest_flag()]
    with tempfile.TemporaryDirectory(prefix="mxq_build_") as tmp:
        objects = [os.path.join(tmp, os.path.splitext(src)[0] + ".o") for src in GPU_SOURCES]
        with concurrent.futures.ThreadPoolExecutor(max_workers=len(GPU_SOURCES)) as pool:
            jobs = [pool.submit(_run, [hipcc, *flags, "-c", "-o", obj, os.path.join(CSRC, src)], verbose)
                    for src, obj in zip(GPU_SOURCES, objects)]
            for job in jobs:
                job.result()
        _run([hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", GPU_LIB, *objects], verbose)
    return GPU_LIB


# floor / rint as instructions (SSE4.1, any x86-64 CPU since 2008) instead of calls into libm; threads
HOST_FLAGS = ["-msse4.1", "-pthread"]


def build_host(verbose=True):
    cmd = [os.path.join(ROCM, "lib", "llvm", "bin", "clang++"), *COMMON, *HOST_FLAGS, _digest_flag(), "-o", HOST_LIB,
           os.path.join(CSRC, "mxq_host.cpp")]
    _run(cmd, verbose)
    return HOST_LIB


def check_sources(verbose=False):
    """Front-end pass (-fsyntax-only, host and gfx950) over every translation unit: seconds instead of
    minutes, and enough to catch a source tree that does not compile (an identifier removed from one
    header and still used by another file)."""
    hipcc = os.path.join(ROCM, "bin", "hipcc")
    flags = ["--offload-arch=gfx950", "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
             *[f for f in COMMON if f != "-shared"], "-fsyntax-only"]
    with concurrent.futures.ThreadPoolExecutor(max_workers=len(GPU_SOURCES)) as pool:
        jobs = [pool.submit(_run, [hipcc, *flags, os.path.join(CSRC, src)], verbose) for src in GPU_SOURCES]
        for job in jobs:
            job.result()
    _run([os.path.join(ROCM, "lib", "llvm", "bin", "clang++"), *[f for f in COMMON if f != "-shared"], *HOST_FLAGS,
          "-fsyntax-only", os.path.join(CSRC, "mxq_host.cpp")], verbose)


def kernel_resources(path=GPU_LIB):
    """What the compiler recorded for every gfx950 kernel of the built library: a list of dicts with
    name, vgprs, agprs, sgprs, lds (static bytes), scratch (bytes of private memory per lane), vgpr_spills,
    sgpr_spills, max_workgroup.  Read from the AMDGPU metadata note of each code object in the library's
    offload bundles (no GPU and no external tool needed) -- the build's own statement of whether a
    kernel spills, how much LDS it declares and how many waves can share a SIMD."""
    import struct
    import msgpack
    with open(path, "rb") as f:
        blob = f.read()
    magic, out, pos = b"__CLANG_OFFLOAD_BUNDLE__", [], 0
    while True:
        start = blob.find(magic, pos)
        if start < 0:
            break
        pos = start + len(magic)
        (n_entries,) = struct.unpack_from("<Q", blob, pos)
        p = pos + 8
        for _ in range(n_entries):
            offset, size, triple_len = struct.unpack_from("<QQQ", blob, p)
            triple = blob[p + 24:p + 24 + triple_len].decode()
            p += 24 + triple_len
            if "gfx950" not in triple or size == 0:
                continue
            elf = blob[start + offset:start + offset + size]
            (shoff,) = struct.unpack_from("<Q", elf, 0x28)
            shentsize, shnum = struct.unpack_from("<HH", elf, 0x3A)
            for k in range(shnum):
                (sh_type,) = struct.unpack_from("<I", elf, shoff + k * shentsize + 4)
                sec_off, sec_size = struct.unpack_from("<QQ", elf, shoff + k * shentsize + 0x18)
                if sh_type != 7:                                         # SHT_NOTE
                    continue
                q = sec_off
                while q < sec_off + sec_size:
                    namesz, descsz, ntype = struct.unpack_from("<III", elf, q)
                    q += 12 + ((namesz + 3) & ~3)
                    desc = elf[q:q + descsz]
                    q += (descsz + 3) & ~3
                    if ntype != 32:                                      # NT_AMDGPU_METADATA
                        continue
                    for kern in msgpack.unpackb(desc, raw=False, strict_map_key=False)["amdhsa.kernels"]:
                        out.append({"name": kern[".name"], "vgprs": kern[".vgpr_count"],
                                    "agprs": kern.get(".agpr_count", 0), "sgprs": kern[".sgpr_count"],
                                    "lds": kern[".group_segment_fixed_size"],
                                    "scratch": kern[".private_segment_fixed_size"],
                                    "vgpr_spills": kern.get(".vgpr_spill_count", 0),
                                    "sgpr_spills": kern.get(".sgpr_spill_count", 0),
                                    "max_workgroup": kern[".max_flat_workgroup_size"]})
    return out


def device_kernels(src_root=ROOT, verbose=False):
    """{mangled kernel name: [instructions]} of the gfx950 code hipcc generates from the sources under
    src_root (a checkout of this repository), every translation unit, with what does not change what a
    kernel does normalized away: branch-label numbers and the offsets at which kernel arguments are loaded."""
    import re
    hipcc = os.path.join(ROCM, "bin", "hipcc")
    csrc = os.path.join(src_root, "microxcaling_amd", "csrc")
    flags = ["--offload-arch=gfx950", "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", "-O3", "-std=c++17",
             "-fPIC", "-ffp-contract=off", "-fvisibility=hidden", "-I" + os.path.join(src_root, "include"), "-I" + csrc,
             "-S", "--cuda-device-only"]
    out = {}
    with tempfile.TemporaryDirectory(prefix="mxq_asm_") as tmp:
        units = [u for u in GPU_SOURCES if os.path.exists(os.path.join(csrc, u))]
        with concurrent.futures.ThreadPoolExecutor(max_workers=len(units)) as pool:
            jobs = [pool.submit(_run, [hipcc, *flags, "-o", os.path.join(tmp, u + ".s"), os.path.join(csrc, u)], verbose)
                    for u in units]
            for job in jobs:
                job.result()
        for u in units:
            name = None
            with open(os.path.join(tmp, u + ".s"), errors="replace") as f:
                for line in f:
                    m = re.match(r"^(_Z\w+):", line)
                    if m:
                        name = m.group(1)
                        out[name] = []
                    elif line.startswith(".Lfunc_end"):
                        name = None
                    elif name is not None:
                        text = line.split(";")[0].strip()
                        if text and not text.startswith("."):
                            text = re.sub(r"\.LBB\d+_", ".LBB_", text)
                            if text.startswith("s_load_dword"):
                                text = re.sub(r"(s\[0:1\]), 0x[0-9a-f]+$", r"\1, <kernarg>", text)
                            out[name].append(text)
    return {k: v for k, v in out.items() if "s_endpgm" in v}  # kernels only (data symbols have no instructions)


def compare_kernels_with(commit, verbose=False):
    """Which kernels' generated code differs between `commit` (its sources are taken from git into a
    temporary folder) and the working tree: {kernel family: [identical, different, only there, only here]}.
    Two builds of a kernel that compare identical execute the same instructions on the same operands; a
    measurement or a test run of the one holds for the other."""
    import collections
    import re
    with tempfile.TemporaryDirectory(prefix="mxq_src_") as tmp:
        tar = subprocess.run(["git", "-C", ROOT, "archive", commit, "microxcaling_amd/csrc", "include"],
                             stdout=subprocess.PIPE, check=True).stdout
        subprocess.run(["tar", "-x", "-C", tmp], input=tar, check=True)
        old = device_kernels(tmp, verbose)
    new = device_kernels(ROOT, verbose)

    def family(name):
        m = re.match(r"_ZN12_GLOBAL__N_1(\d+)", name)
        return name[m.end():m.end() + int(m.group(1))] if m else name
    table = collections.defaultdict(lambda: [0, 0, 0, 0])
    for name, code in old.items():
        table[family(name)][2 if name not in new else 0 if new[name] == code else 1] += 1
    for name in new:
        if name not in old:
            table[family(name)][3] += 1
    return dict(table)


def build_all(verbose=True):
    return build_gpu(verbose), build_host(verbose)


if __name__ == "__main__":
    if len(sys.argv) == 3 and sys.argv[1] == "--compare-with":
        # python -m microxcaling_amd.build_ext --compare-with <commit>: generated code, kernel by kernel
        print("%-34s %9s %9s %10s %9s" % ("kernel", "identical", "different", "only there", "only here"))
        for fam, row in sorted(compare_kernels_with(sys.argv[2]).items()):
            print("%-34s %9d %9d %10d %9d" % (fam, *row))
    else:
        build_all(verbose=True)
        print("built", GPU_LIB, HOST_LIB)
