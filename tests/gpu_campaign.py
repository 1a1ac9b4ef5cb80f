"""Random-program campaign: for a number of seconds, draw random race-free programs (2 to 64 ranks,
six dtypes, 700 to 400,003 elements, 10 to 120 ops of any size and alignment, sum / max / min) and
run each through every runner (level and persistent runners at the automatic and at the smallest
item size, auto mode, and for position-aligned programs the slot and the register column runners)
against the CPU oracle, bit for bit.  Not collected by pytest (it runs as long as it is told to):

    python tests/gpu_campaign.py <seed> <seconds>

prints every case before it runs and "campaign ok: N programs" at the end; exit status 1 at the
first mismatch."""
import sys, time
import os
sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
import torch
from helpers import bits_equal, mismatch_report, oracle_buffers, random_program, seeded_inputs
from pccl_amd.engine import Engine
DTYPES = ["float32", "bfloat16", "int32", "float16", "float8_e4m3", "float8_e5m2"]
import numpy as np
rng = np.random.default_rng(int(sys.argv[1]) if len(sys.argv) > 1 else 0)
t_end = time.time() + float(sys.argv[2]) if len(sys.argv) > 2 else time.time() + 120
count = 0
while time.time() < t_end:
    seed = int(rng.integers(1 << 30))
    world = int(rng.choice([2, 3, 5, 8, 9, 16, 17, 24, 33, 48, 64]))
    dtype = DTYPES[int(rng.integers(len(DTYPES)))]
    n = int(rng.choice([700, 4099, 20011, 65536, 150001, 400003]))
    ops = int(rng.integers(10, 120))
    aligned = bool(rng.integers(2))
    red = ("sum",) if dtype.startswith("float8") else ("sum", "max", "min")
    jsons = random_program(seed, world, n, ops, dtype, aligned, reduce_ops=red)
    x = seeded_inputs("randint" if dtype == "int32" else "randn", world, n, dtype, seed=seed % 1000)
    want = oracle_buffers(jsons, x, dtype)
    eng = Engine(world, 0)
    for r, j in enumerate(jsons): eng.register_operation_json("rnd", j, r)
    modes = ["stepwise", "persistent", "auto"] + (["column", "column-reg"] if aligned else [])
    for mode in modes:
        print(f"case seed={seed} R={world} {dtype} n={n} ops={ops} aligned={aligned} mode={mode}", flush=True)
        if mode == "column-reg":
            eng.set_option("mode", "column"); eng.set_option("lds_slots", 0)
        else:
            eng.set_option("lds_slots", 1); eng.set_option("mode", mode)
        for tb in ((0, 4096) if mode in ("stepwise", "persistent") else (0,)):
            eng.set_option("step_tile_bytes", tb)
            bufs = [t.cuda() for t in x]
            eng.execute_inplace("rnd", bufs, sync=True)
            for r in range(world):
                if not bits_equal(bufs[r], want[r]):
                    print("MISMATCH", mode, tb, r, mismatch_report(bufs[r], want[r]), flush=True); sys.exit(1)
    eng.close(); count += 1
print("campaign ok:", count, "programs")
