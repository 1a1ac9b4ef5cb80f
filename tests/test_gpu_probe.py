"""The memory-system probe behind the ceilings under profiles/ (pccl_amd/csrc/stream_probe.hip, run
through `bench.py --probe`): every kind of case on a small size, each one's result checked by the
probe itself on the host.  The probe is a measuring tool and not part of the library; this keeps it
building and computing what it says."""
import json
import os
import subprocess
import sys

import pytest

from pccl_amd import build as lib_build

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))

CASES = ("read:256 write:256 copy:256 tile:256:2:8:0 tile:256:1:8:1 tile:256:2:4:0 "
         "phased:512:16:4:0:0 phased:512:16:4:1:0 phased:512:16:4:2:0 phased:256:32:8:1:1 phased:256:32:8:1:2 phased:512:16:4:1:2 "
         "phased:256:32:8:1:3 phased:256:32:8:1:4 phased:256:32:8:1:5 phased:512:16:4:1:3 "
         "sweeps:0:0 sweeps:1:0 sweeps:2:0 sweeps:3:0 sweeps:1:1 sweeps:2:1 sweeps:3:1")


def test_every_kind_of_case_runs_and_checks_its_result():
    assert os.path.exists(lib_build.PROBE), "the probe is built by pccl_amd/build.py"
    # 8 ranks x 96 MiB: three sweeps of the persistent shapes on a 256-CU GPU, so that groups of two and
    # three sweeps have a remainder
    out = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--probe", "8 100663296 " + CASES],
                         capture_output=True, text=True, timeout=170)
    assert out.returncode == 0, out.stderr[-2000:]
    rows = [json.loads(line) for line in out.stdout.splitlines() if line.startswith("{")]
    assert [r["case"] for r in rows] == CASES.split()
    for r in rows:
        assert "error" not in r, r
        assert r["verified"] is True, r
        assert 0.0 < r["frac_of_8TBps"] < 1.0, r
    unknown = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--probe", "8 100663296 sweeps:4:0 nothing:1"],
                             capture_output=True, text=True, timeout=120)
    rows = [json.loads(line) for line in unknown.stdout.splitlines() if line.startswith("{")]
    assert len(rows) == 2 and all("error" in r for r in rows)
