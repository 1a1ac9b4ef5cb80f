"""Collective campaign: for a number of seconds, draw collectives from the schedule templates (ring /
recursive halving-doubling / tree allreduce, ring reduce_scatter, allgather and alltoall; 2 to 32
ranks, 1 to 4 channels, five dtypes, sum / max / min where the dtype has them) and run each as a
staged call (separate input and output tensors, the reference's call shape) and, for allreduce, in
place, in every runner mode and with the staging fused into the program or not, against the CPU
oracle, bit for bit.  Not collected by pytest:

    python tests/gpu_campaign_collectives.py <seed> <seconds>
"""
import os
import sys
import time

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
import numpy as np
import torch
from helpers import bits_equal, graph_jsons, mismatch_report, oracle_buffers, seeded_inputs
from pccl_amd.engine import Engine

DTYPES = ["float32", "bfloat16", "float16", "int32", "float8_e4m3"]
rng = np.random.default_rng(int(sys.argv[1]) if len(sys.argv) > 1 else 0)
t_end = time.time() + (float(sys.argv[2]) if len(sys.argv) > 2 else 120.0)
count = 0


def fail(what, got, want):
    print("MISMATCH", what, mismatch_report(got, want), flush=True)
    sys.exit(1)


while time.time() < t_end:
    kind = str(rng.choice(["ring_ar", "rhd_ar", "tree_ar", "ring_rs", "ring_ag", "ring_a2a"]))
    pow2 = kind in ("rhd_ar", "tree_ar")
    world = int(rng.choice([2, 4, 8, 16, 32] if pow2 else [2, 3, 4, 6, 8, 12, 16, 24, 32]))
    channels = 1 if kind in ("rhd_ar", "tree_ar", "ring_a2a") else int(rng.choice([1, 2, 4]))
    dtype = DTYPES[int(rng.integers(len(DTYPES)))]
    unit = world * channels
    n = unit * int(rng.choice([1, 3, 16, 129, 1000, 4099]))
    red = "sum" if dtype.startswith("float8") or kind in ("ring_rs", "ring_ag", "ring_a2a") else str(rng.choice(["sum", "max", "min"]))
    ext = {"reduce_op": red} if kind.endswith("_ar") and red != "sum" else {}
    alg, method = {"ring_ar": ("ring", "build_allreduce"), "rhd_ar": ("rhd", "build_allreduce"), "tree_ar": ("tree", "build_allreduce"),
                   "ring_rs": ("ring", "build_reduce_scatter"), "ring_ag": ("ring", "build_allgather"), "ring_a2a": ("ring", "build_alltoall")}[kind]
    seed = int(rng.integers(1000))
    src_kind = "randint" if dtype == "int32" else "randn"
    print(f"case {kind} R={world} ch={channels} {dtype} n={n} {red} seed={seed}", flush=True)
    jsons = graph_jsons(alg, method, world, n, dtype, "sm", channels, **ext)
    chunk = n // world
    if kind == "ring_ag":
        x = seeded_inputs(src_kind, world, chunk, dtype, seed=seed)
        want = oracle_buffers(jsons, x, dtype, place=lambda r: r * chunk, buffer_elems=n)
    else:
        x = seeded_inputs(src_kind, world, n, dtype, seed=seed)
        want = oracle_buffers(jsons, x, dtype, buffer_elems=2 * n if kind == "ring_a2a" else 0)
    eng = Engine(world, 0)
    for r, j in enumerate(jsons):
        eng.register_operation_json("op", j, r)
    for mode in ("auto", "stepwise", "persistent"):
        for fuse in (1, 0):
            eng.set_option("mode", mode)
            eng.set_option("fuse_staging", fuse)
            ins = [t.cuda() for t in x]
            out_elems = chunk if kind == "ring_rs" else n
            outs = [torch.zeros(out_elems, dtype=ins[0].dtype, device="cuda") for _ in range(world)]
            eng.execute_operation("op", ins, outs)
            for r in range(world):
                if not bits_equal(ins[r], x[r]):
                    fail(f"{mode} fuse={fuse}: input of rank {r} was modified", ins[r], x[r])
                if kind.endswith("_ar"):
                    if not bits_equal(outs[r], want[r][:n]):
                        fail(f"{mode} fuse={fuse} staged rank {r}", outs[r], want[r][:n])
                elif kind == "ring_rs":
                    if not bits_equal(outs[r], want[r][r * chunk:(r + 1) * chunk]):
                        fail(f"{mode} fuse={fuse} reduce_scatter rank {r}", outs[r], want[r][r * chunk:(r + 1) * chunk])
                elif kind == "ring_ag":
                    if channels == 1 and not bits_equal(outs[r], torch.cat(x)):
                        fail(f"{mode} fuse={fuse} allgather rank {r}", outs[r], torch.cat(x))
                else:
                    exp = torch.cat([x[i][r * chunk:(r + 1) * chunk] for i in range(world)])
                    if not bits_equal(outs[r], exp):
                        fail(f"{mode} fuse={fuse} alltoall rank {r}", outs[r], exp)
        if kind.endswith("_ar"):
            bufs = [t.cuda() for t in x]
            eng.execute_inplace("op", bufs, sync=True)
            for r in range(world):
                if not bits_equal(bufs[r], want[r][:n]):
                    fail(f"{mode} in place rank {r}", bufs[r], want[r][:n])
    eng.close()
    count += 1
print("campaign ok:", count, "collectives")
