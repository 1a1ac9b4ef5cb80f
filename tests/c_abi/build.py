"""Builds the two stand-alone clients of the C ABI against include/pccl_hip.h and the built library:
ring_client.c with the C compiler (the header must compile as C) and adapter_check.cc with the C++
compiler.  Both link only libpccl_hip.so and libamdhip64."""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
OUT = os.path.join(HERE, "build", "ring_client")
ADAPTER = os.path.join(HERE, "build", "adapter_check")


def build() -> str:
    os.makedirs(os.path.dirname(OUT), exist_ok=True)
    lib_dir = os.path.join(ROOT, "pccl_amd", "lib")
    common = ["-O2", "-Wall", "-Wextra", "-Werror", "-D__HIP_PLATFORM_AMD__",
              "-I", os.path.join(ROOT, "include"), "-I/opt/rocm/include"]
    link = ["-L", lib_dir, "-lpccl_hip", "-L/opt/rocm/lib", "-lamdhip64",
            "-Wl,-rpath,$ORIGIN/../../../pccl_amd/lib", "-Wl,-rpath,/opt/rocm/lib"]
    subprocess.run(["gcc", "-std=c11"] + common + [os.path.join(HERE, "ring_client.c"), "-o", OUT] + link, check=True)
    subprocess.run(["g++", "-std=c++17"] + common + [os.path.join(HERE, "adapter_check.cc"), "-o", ADAPTER] + link, check=True)
    return OUT


if __name__ == "__main__":
    print(build())
    sys.exit(0)
