"""The memory-system probe behind the vector-width and stream-count tables (tests/probes/): its
quick half runs here so that the command the tables were made with keeps working."""
import os
import re
import subprocess

import pytest

from helpers import ROOT

PROBE = os.path.join(ROOT, "tests", "probes", "build", "stream_probe")


@pytest.mark.gpu
def test_width_probe_runs_and_reports_three_rates():
    if not os.path.exists(PROBE):
        from tests.probes import build          # not built yet (build() of the entry module does it)
        build.build()
    print("stream_probe width", flush=True)
    p = subprocess.run([PROBE, "width"], capture_output=True, text=True, timeout=120)
    assert p.returncode == 0, p.stdout + p.stderr
    rates = [float(m) for m in re.findall(r"(\d+) GB/s", p.stdout)]
    assert len(rates) == 3 and all(1000.0 < r < 8000.0 for r in rates), p.stdout
