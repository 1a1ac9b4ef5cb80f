"""Build pccl_amd/lib/libpccl_hip.so: host logic + gfx950 kernels in one shared library.

hipcc cross-compiles for gfx950 without a GPU.  ``-packed-fp32-ops`` is switched off for all
device code: the compiler must not fuse float adds into packed-FP32 instructions here.
"""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OUT_DIR = os.path.join(HERE, "lib")
OUT = os.path.join(OUT_DIR, "libpccl_hip.so")
SOURCES = ["graph.cc", "program.cc", "capi.cc", "kernels.hip"]
HEADERS = ["graph.h", "program.h", "kernels.h", "json_min.h", "../../include/pccl_hip.h", "stream_probe.hip"]


def is_stale() -> bool:
    if not os.path.exists(OUT):
        return True
    t = os.path.getmtime(OUT)
    return any(os.path.getmtime(os.path.join(CSRC, f)) > t for f in SOURCES + HEADERS)


def build(force: bool = True, verbose: bool = False) -> str:
    if not force and not is_stale():
        return OUT
    os.makedirs(OUT_DIR, exist_ok=True)
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    common = ["-O3", "-std=c++17", "-fPIC", "--offload-arch=gfx950", "-Wall", "-Wno-unused-function",
              "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]
    objs = []
    procs = []
    for src in SOURCES:
        obj = os.path.join(OUT_DIR, src.replace(".", "_") + ".o")
        objs.append(obj)
        if src.endswith(".hip"):
            cmd = [hipcc] + common + ["-x", "hip", "-c", os.path.join(CSRC, src), "-o", obj]
        else:  # host-only translation units: plain C++ against the HIP runtime API headers
            cmd = [hipcc, "-O3", "-std=c++17", "-fPIC", "-Wall", "-x", "c++", "-D__HIP_PLATFORM_AMD__",
                   "-I/opt/rocm/include", "-c", os.path.join(CSRC, src), "-o", obj]
        if verbose:
            print(" ".join(cmd))
        procs.append((src, subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT)))
    failed = False
    for src, p in procs:
        out, _ = p.communicate()
        text = "\n".join(l for l in out.decode().splitlines()
                         if "packed-fp32-ops' is not a recognized feature" not in l)
        if p.returncode != 0:
            failed = True
            sys.stderr.write(f"--- {src} failed ---\n{text}\n")
        elif verbose and text.strip():
            print(text)
    if failed:
        raise RuntimeError("hipcc failed")
    subprocess.run([hipcc, "-shared", "-fPIC", "--offload-arch=gfx950", "-o", OUT] + objs, check=True)
    build_probe(hipcc, common)
    return OUT


PROBE = os.path.join(OUT_DIR, "stream_probe")


def build_probe(hipcc: str, common) -> str:
    """The memory-system probe (bare kernels of the runners' traffic shapes; `bench.py --probe`): a
    standalone program, not part of the library."""
    cmd = [hipcc] + [c for c in common if c != "-fPIC"] + [os.path.join(CSRC, "stream_probe.hip"), "-o", PROBE]
    out = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT)
    if out.returncode != 0:
        sys.stderr.write(out.stdout.decode())
        raise RuntimeError("hipcc failed on stream_probe.hip")
    return PROBE


if __name__ == "__main__":
    print(build(force="--if-stale" not in sys.argv, verbose="-v" in sys.argv))
