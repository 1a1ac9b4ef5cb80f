"""The C ABI used from plain C (tests/c_abi/ring_client.c): compiled with gcc against
include/pccl_hip.h, linked to libpccl_hip.so and libamdhip64 only."""
import os
import subprocess

import pytest

from helpers import ROOT

CLIENT = os.path.join(ROOT, "tests", "c_abi", "build", "ring_client")
GRAPHS = os.path.join(ROOT, "tests", "golden", "graphs")


def client():
    if not os.path.exists(CLIENT):
        from tests.c_abi import build          # not built yet (build() of the entry module does it)
        build.build()
    return CLIENT


def test_header_compiles_as_c_and_the_client_links():
    """No arguments: the program prints its usage and leaves before any HIP call, which still takes
    the dynamic loader through libpccl_hip.so and libamdhip64."""
    p = subprocess.run([client()], capture_output=True, text=True, timeout=60)
    assert p.returncode == 2 and "usage" in p.stderr


@pytest.mark.gpu
@pytest.mark.parametrize("stem,world,n", [("ring_ar_sm_w2_n2048_bf16_c1", 2, 2048), ("ring_ar_tma_w8_n8192_bf16_c4", 8, 8192)])
def test_ring_allreduce_from_plain_c(stem, world, n):
    """Registers the reference emitter's graph files, runs the staged call and the in-place call in
    all three runner modes and checks the closed form R (R + 1) / 2 (reference
    tests/test_correctness.py:142,170-171)."""
    files = [os.path.join(GRAPHS, f"{stem}_rank{r}.json") for r in range(world)]
    p = subprocess.run([client(), str(n)] + files, capture_output=True, text=True, timeout=120)
    assert p.returncode == 0, p.stdout + p.stderr
    assert f"ok ranks={world} elements={n}" in p.stdout
