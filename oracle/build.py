"""Compile the CPU oracle (oracle/pccl_oracle.c) into oracle/libpccl_oracle.so.

Test infrastructure only.  The reference's own implementation of this path is CUDA-only
(nvcc, <cuda.h>, inline PTX, un-vendored nlohmann/spdlog submodules), so there is no
``oracle/_ref`` build: nothing of the reference compiles in a ROCm image.
"""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
SRC = os.path.join(HERE, "pccl_oracle.c")
OUT = os.path.join(HERE, "libpccl_oracle.so")


def build(force: bool = True) -> str:
    if not force and os.path.exists(OUT) and os.path.getmtime(OUT) >= os.path.getmtime(SRC):
        return OUT
    # -ffp-contract=off / no fast-math: the element loops must stay plain IEEE adds.
    # -mavx2 only: the library is built here and run on the GPU box's host CPU.
    cmd = ["gcc", "-O3", "-mavx2", "-fopenmp", "-ffp-contract=off", "-fno-fast-math",
           "-shared", "-fPIC", "-Wall", "-o", OUT, SRC]
    subprocess.run(cmd, check=True)
    return OUT


if __name__ == "__main__":
    print(build(force="--if-stale" not in sys.argv))
