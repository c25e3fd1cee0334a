"""Builds the CPU checker (oracle/libcgpt_oracle.so) with gcc.

TEST INFRASTRUCTURE — not part of the product. Flags are the reference's CPU
build flags (CMakeLists.txt:19-22, 63-66): -O2 -fopenmp -mavx2 -mfma -mf16c.

oracle/_ref (a build of the reference's own CPU sources) is not produced: every
reference CPU source includes <cuda_runtime.h> and <cublasLt.h> through
include/core/tensor.h:9 and include/core/dtype.h:3, and this image has neither,
so the reference is unbuildable here without writing stand-in headers.
"""
from __future__ import annotations

import pathlib
import subprocess

HERE = pathlib.Path(__file__).resolve().parent
LIB = HERE / "libcgpt_oracle.so"


def build() -> pathlib.Path:
    cmd = ["gcc", "-O2", "-fopenmp", "-mavx2", "-mfma", "-mf16c", "-fPIC", "-shared", "-std=c11",
           "-ffp-contract=off", "-Wall", "-o", str(LIB), str(HERE / "cgpt_cpu_ops.c"), "-lm"]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError(f"gcc failed:\n{proc.stderr}")
    return LIB


if __name__ == "__main__":
    print(build())
