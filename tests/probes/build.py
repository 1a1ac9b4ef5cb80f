"""Builds tests/probes/stream_probe.hip for gfx950 into tests/probes/build/stream_probe (a standalone
program: HIP runtime only, not linked to the library)."""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
OUT = os.path.join(HERE, "build", "stream_probe")


def build() -> str:
    os.makedirs(os.path.dirname(OUT), exist_ok=True)
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    cmd = [hipcc, "-O3", "-std=c++17", "--offload-arch=gfx950", "-Wall",
           "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
           os.path.join(HERE, "stream_probe.hip"), "-o", OUT]
    subprocess.run(cmd, check=True)
    return OUT


if __name__ == "__main__":
    print(build())
    sys.exit(0)
