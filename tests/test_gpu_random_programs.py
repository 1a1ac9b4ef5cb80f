"""Random race-free programs through every runner against the oracle.

The programs come from helpers.random_program: random ranks, peers, element ranges of any size and
alignment, sum / max / min, in one global order enforced by notify / wait pairs.  The linker turns
each into conflict-based dependency levels; the level runner, the persistent flag-ordered runner
and (for position-aligned programs) the column runner must all reproduce the oracle's buffers bit
for bit.
"""
import pytest
import torch

from helpers import bits_equal, mismatch_report, oracle_buffers, random_program, seeded_inputs

pytestmark = pytest.mark.gpu

DTYPES = ["float32", "bfloat16", "int32", "float16", "float8_e4m3"]


@pytest.mark.parametrize("seed", range(10))
@pytest.mark.parametrize("aligned", [True, False], ids=["aligned", "general"])
def test_random_program_all_runners(engine_factory, seed, aligned):
    world = 2 + seed % 6
    dtype = DTYPES[seed % len(DTYPES)]
    n = 3000 + 517 * seed                     # odd sizes: heads, tails, cut vectors
    red = ("sum",) if dtype.startswith("float8") else ("sum", "max", "min")
    jsons = random_program(1000 + seed, world, n, 40 + 6 * seed, dtype, aligned, reduce_ops=red)
    kind = "randint" if dtype == "int32" else "randn"
    x = seeded_inputs(kind, world, n, dtype, seed=seed)
    want = oracle_buffers(jsons, x, dtype)
    engine = engine_factory(world)
    for r, j in enumerate(jsons):
        engine.register_operation_json("rnd", j, r)
    info = engine.op_info("rnd")
    assert info["position_aligned"] == int(aligned) and info["residual_signals"] == 0
    modes = ["stepwise", "persistent", "auto"] + (["column"] if aligned else [])
    for mode in modes:
        print(f"seed {seed} {dtype} R={world} n={n} aligned={aligned} mode={mode}", flush=True)
        engine.set_option("mode", mode)
        bufs = [t.cuda() for t in x]
        engine.execute_inplace("rnd", bufs, sync=True)
        for r in range(world):
            assert bits_equal(bufs[r], want[r]), f"{mode}, rank {r}: {mismatch_report(bufs[r], want[r])}"
    if aligned:     # the register runner too
        engine.set_option("mode", "column")
        engine.set_option("lds_slots", 0)
        bufs = [t.cuda() for t in x]
        engine.execute_inplace("rnd", bufs, sync=True)
        engine.set_option("lds_slots", 1)
        for r in range(world):
            assert bits_equal(bufs[r], want[r]), f"register runner, rank {r}: {mismatch_report(bufs[r], want[r])}"
    engine.set_option("mode", "auto")
