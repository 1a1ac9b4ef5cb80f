"""Builds tests/c_abi/ring_client.c with the C compiler against include/pccl_hip.h and the built
library.  The header must compile as C; the program links only libpccl_hip.so and libamdhip64."""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
OUT = os.path.join(HERE, "build", "ring_client")


def build() -> str:
    os.makedirs(os.path.dirname(OUT), exist_ok=True)
    lib_dir = os.path.join(ROOT, "pccl_amd", "lib")
    cmd = ["gcc", "-std=c11", "-O2", "-Wall", "-Wextra", "-Werror", "-D__HIP_PLATFORM_AMD__",
           "-I", os.path.join(ROOT, "include"), "-I/opt/rocm/include",
           os.path.join(HERE, "ring_client.c"), "-o", OUT,
           "-L", lib_dir, "-lpccl_hip", "-L/opt/rocm/lib", "-lamdhip64",
           "-Wl,-rpath,$ORIGIN/../../../pccl_amd/lib", "-Wl,-rpath,/opt/rocm/lib"]
    subprocess.run(cmd, check=True)
    return OUT


if __name__ == "__main__":
    print(build())
    sys.exit(0)
