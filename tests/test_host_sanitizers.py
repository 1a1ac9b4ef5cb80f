"""The host-only sources (graph loader, linker) built with AddressSanitizer and
UndefinedBehaviorSanitizer and driven over clean and damaged graph documents
(tests/sanitize/fuzz_driver.cc).  Host code only: no HIP call is compiled in."""
import os
import shutil
import subprocess

import pytest

from helpers import ROOT

CSRC = os.path.join(ROOT, "pccl_amd", "csrc")
GRAPHS = os.path.join(ROOT, "tests", "golden", "graphs")


@pytest.mark.skipif(shutil.which("g++") is None, reason="needs g++")
def test_loader_and_linker_under_asan_and_ubsan(tmp_path):
    exe = str(tmp_path / "fuzz_driver")
    cmd = ["g++", "-std=c++17", "-O1", "-g", "-fsanitize=address,undefined", "-fno-sanitize-recover=undefined",
           "-static-libasan", "-static-libubsan", "-D__HIP_PLATFORM_AMD__", "-I", CSRC, "-I", os.path.join(ROOT, "include"),
           "-I/opt/rocm/include", os.path.join(ROOT, "tests", "sanitize", "fuzz_driver.cc"),
           os.path.join(CSRC, "graph.cc"), os.path.join(CSRC, "program.cc"), "-o", exe]
    build = subprocess.run(cmd, capture_output=True, text=True, timeout=300)
    assert build.returncode == 0, build.stderr[-3000:]
    cases = [("ring_ar_sm_w2_n2048_bf16_c1", 2), ("ring_ar_sm_w4_n4096_f32_c2", 4), ("tree_ar_sm_w8_n1024_f32_c1", 8),
             ("rhd_ar_sm_w8_n4096_f32_c1", 8), ("ring_a2a_sm_w4_n4096_bf16_c1", 4), ("ring_rs_sm_w4_n4096_f16_c1", 4)]
    args = []
    for stem, world in cases:
        args += [os.path.join(GRAPHS, stem), str(world)]
    env = dict(os.environ, ASAN_OPTIONS="detect_leaks=1:abort_on_error=0", UBSAN_OPTIONS="print_stacktrace=1")
    run = subprocess.run([exe] + args + ["--trials", "120"], capture_output=True, text=True, timeout=600, env=env)
    assert run.returncode == 0, (run.stdout + run.stderr)[-4000:]
    assert "ERROR: AddressSanitizer" not in run.stderr and "runtime error" not in run.stderr, run.stderr[-4000:]
    counts = dict(zip(run.stdout.split()[0::2], map(int, run.stdout.split()[1::2])))
    assert counts["failed"] > 100 and counts["loaded"] > 20 and counts["linked"] >= 3 * len(cases)
