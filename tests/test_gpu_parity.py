"""GPU parity: the HIP executor against the CPU oracle, bit for bit, through the C ABI.

Every case runs in the three execution modes — column (position-decomposed, no inter-workgroup
ordering), stepwise (one launch per dependency level) and persistent (one launch, device-side
flags with bounded waits) — in place on the caller's buffers and staged (separate input/output
tensors, the reference's call shape).
"""
import pytest
import torch

from helpers import (TORCH_DTYPE, bits_equal, graph_jsons, mismatch_report, oracle_buffers,
                     seeded_inputs)

pytestmark = pytest.mark.gpu

_counter = [0]


def run_gpu(engine, jsons, inputs, mode, inplace=False, out_elems=None):
    _counter[0] += 1
    name = f"op{_counter[0]}"
    for r, j in enumerate(jsons):
        engine.register_operation_json(name, j, r)
    engine.set_option("mode", mode)
    dev = [x.cuda() for x in inputs]
    if inplace:
        engine.execute_inplace(name, dev, sync=True)
        return [d.cpu() for d in dev], engine.op_info(name)
    outs = None
    if out_elems is not None:
        outs = [torch.zeros(out_elems, dtype=inputs[0].dtype, device="cuda") for _ in inputs]
    outs = engine.execute_operation(name, dev, outs)
    return [o.cpu() for o in outs], engine.op_info(name)


CASES = [
    # alg, world, n, dtype, channels, input kind
    ("ring", 8, 1024 * 1024, "float32", 1, "randn"),       # configuration 1 (plumbing)
    ("ring", 8, 1 << 20, "bfloat16", 4, "randn"),          # headline shape, scaled down
    ("ring", 2, 2048, "bfloat16", 1, "rank+1"),
    ("ring", 3, 3 * 4096, "float16", 2, "randn0.1"),       # non power-of-two world
    ("rhd", 16, 1 << 18, "float32", 2, "uniform"),         # configuration 3, scaled down
    ("rhd", 4, 4096, "bfloat16", 1, "randn"),
    ("tree", 32, 1 << 16, "float32", 1, "randn"),
    ("tree", 8, 8192, "float16", 1, "randn0.1"),
]


PERSISTENT_OFF = pytest.mark.skip(reason="the persistent flag-ordered runner hung on MI355X (wait for a "
                                   "predecessor's tile counter never returned); the mode is refused "
                                   "by the library until the cause is found")
MODES = ["column", "stepwise", pytest.param("persistent", marks=PERSISTENT_OFF)]


@pytest.mark.parametrize("alg,world,n,dtype,channels,kind", CASES)
@pytest.mark.parametrize("mode", MODES)
def test_allreduce_matches_oracle(engine_factory, alg, world, n, dtype, channels, kind, mode):
    print(f"case {alg} R={world} n={n} {dtype} ch={channels} mode={mode}", flush=True)
    jsons = graph_jsons(alg, "build_allreduce", world, n, dtype, "sm", channels)
    inputs = seeded_inputs(kind, world, n, dtype)
    expect = oracle_buffers(jsons, inputs, dtype)
    engine = engine_factory(world)
    print("  in place", flush=True)
    got, info = run_gpu(engine, jsons, inputs, mode, inplace=True)
    assert info["residual_signals"] == 0
    for r in range(world):
        assert bits_equal(got[r], expect[r]), f"in place, rank {r}: {mismatch_report(got[r], expect[r])}"
    print("  staged", flush=True)
    got2, _ = run_gpu(engine, jsons, inputs, mode)
    for r in range(world):
        assert bits_equal(got2[r], expect[r]), f"staged, rank {r}: {mismatch_report(got2[r], expect[r])}"


@pytest.mark.parametrize("mode", MODES)
def test_closed_form_rank_plus_one(engine_factory, mode):
    """Input rank+1 everywhere -> allreduce = R(R+1)/2, exact in bf16
    (reference tests/test_correctness.py:142,170-171)."""
    world, n = 8, 1 << 16
    jsons = graph_jsons("ring", "build_allreduce", world, n, "bfloat16", "tma", 1)
    inputs = seeded_inputs("rank+1", world, n, "bfloat16")
    got, _ = run_gpu(engine_factory(world), jsons, inputs, mode)
    for r in range(world):
        assert torch.all(got[r].float() == world * (world + 1) / 2)


@pytest.mark.parametrize("mode", MODES)
def test_reduce_scatter_and_allgather(engine_factory, mode):
    """reference tests/test_correctness.py:196-241: reduce_scatter output is one chunk of sums;
    allgather input is one chunk, output the concatenation."""
    world, n = 8, 1 << 16
    chunk = n // world
    engine = engine_factory(world)
    jsons = graph_jsons("ring", "build_reduce_scatter", world, n, "float16", "tma", 1)
    inputs = seeded_inputs("randn0.1", world, n, "float16")
    expect = oracle_buffers(jsons, inputs, "float16")
    got, _ = run_gpu(engine, jsons, inputs, mode, out_elems=chunk)
    for r in range(world):
        assert bits_equal(got[r], expect[r][r * chunk:(r + 1) * chunk]), mismatch_report(got[r], expect[r][r * chunk:(r + 1) * chunk])

    jsons = graph_jsons("ring", "build_allgather", world, n, "float16", "tma", 1)
    parts = seeded_inputs("randn0.1", world, chunk, "float16", seed=1)
    got, _ = run_gpu(engine, jsons, parts, mode, out_elems=n)
    whole = torch.cat(parts)
    for r in range(world):
        assert bits_equal(got[r], whole), f"rank {r}: {mismatch_report(got[r], whole)}"


@pytest.mark.parametrize("mode", ["stepwise", pytest.param("persistent", marks=PERSISTENT_OFF)])
def test_alltoall(engine_factory, mode):
    """reference tests/test_correctness.py:243-272: out[i] chunk = chunk r of rank i's input."""
    world, n = 4, 1 << 12
    chunk = n // world
    jsons = graph_jsons("ring", "build_alltoall", world, n, "bfloat16", "tma", 1)
    inputs = [torch.cat([torch.full((chunk,), r * 100 + i, dtype=torch.bfloat16) for i in range(world)])
              for r in range(world)]
    got, info = run_gpu(engine_factory(world), jsons, inputs, mode)
    assert info["position_aligned"] == 0
    for r in range(world):
        want = torch.cat([torch.full((chunk,), i * 100 + r, dtype=torch.bfloat16) for i in range(world)])
        assert bits_equal(got[r], want), mismatch_report(got[r], want)


def test_persistent_mode_is_refused(engine_factory):
    from pccl_amd._lib import PcclError, ERR_UNSUPPORTED
    engine = engine_factory(2)
    with pytest.raises(PcclError) as e:
        engine.set_option("mode", "persistent")
    assert e.value.code == ERR_UNSUPPORTED
    engine.set_option("mode", "auto")
