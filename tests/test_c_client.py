"""The C ABI used from plain C (tests/c_abi/ring_client.c, compiled with gcc) and from a stand-alone
C++ translation unit that lays its trigger arrays out with the reference's own struct declarations
(tests/c_abi/adapter_check.cc); both link libpccl_hip.so and libamdhip64 only."""
import os
import subprocess

import pytest

from helpers import ROOT

CLIENT = os.path.join(ROOT, "tests", "c_abi", "build", "ring_client")
ADAPTER = os.path.join(ROOT, "tests", "c_abi", "build", "adapter_check")
GRAPHS = os.path.join(ROOT, "tests", "golden", "graphs")


def client():
    if not os.path.exists(CLIENT) or not os.path.exists(ADAPTER):
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


@pytest.mark.gpu
def test_trigger_arrays_laid_out_by_the_reference_headers():
    """The row of the drop-in boundary that no loader of this repository touches: arrays built from
    struct declarations with the reference's field order (proxy_trigger.h:8-30, primitive.h:8-17)
    go through pccl_hip_register_triggers and pccl_hip_execute in all three modes and give the closed
    form R (R + 1) / 2."""
    client()
    p = subprocess.run([ADAPTER], capture_output=True, text=True, timeout=120)
    assert p.returncode == 0, p.stdout + p.stderr
    assert "ok triggers laid out by the reference's headers: ranks=2 elements=2048 result=3" in p.stdout
