"""Compiles the oracle's C restatement (mxq_oracle.c) into oracle/libmxq_oracle.so with gcc.

The reference's own C++ (mx/cpp/funcs.cpp and headers) is not built: it includes CUDA and torch
extension headers (cuda.h, cuda_bf16.h, cublas_v2.h, torch/extension.h) that are absent here, so
there is no oracle/_ref."""
import os
import subprocess

HERE = os.path.dirname(os.path.abspath(__file__))
LIB = os.path.join(HERE, "libmxq_oracle.so")


def build(verbose=True):
    cmd = ["gcc", "-O2", "-std=c11", "-fPIC", "-shared", "-ffp-contract=off", "-fno-fast-math",
           "-o", LIB, os.path.join(HERE, "mxq_oracle.c"), "-lm"]
    if verbose:
        print(" ".join(cmd), flush=True)
    subprocess.run(cmd, check=True)
    return LIB


if __name__ == "__main__":
    build()
