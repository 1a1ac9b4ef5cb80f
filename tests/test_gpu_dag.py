"""Graphs that are not single chains, through the level-scheduled runner, the persistent
flag-ordered runner and (where the ops are position-aligned) the column runner: Pipeline-built graphs, fork / join over streams with several
dependencies and successors per op, and `noop` nodes — the ground the reference covers with its
DAG kernel (cuda_executor.cu:526-918: remaining_deps counters, up to 8 successors per op).
"""
import json

import pytest
import torch

from helpers import (bits_equal, graph_jsons, mismatch_report, oracle_buffers, pipelined_ring_allreduce,
                     seeded_inputs)
from pccl_amd.dsl import CommunicationOp, Stream, compile_to_json_string

pytestmark = pytest.mark.gpu


def run(engine, name, jsons, inputs, mode):
    for r, j in enumerate(jsons):
        engine.register_operation_json(name, j, r)
    engine.set_option("mode", mode)
    dev = [x.cuda() for x in inputs]
    engine.execute_inplace(name, dev, sync=True)
    return [d.cpu() for d in dev]


@pytest.mark.parametrize("world,depth,dtype", [(4, 2, "float32"), (8, 3, "bfloat16"), (3, 3, "float16")])
@pytest.mark.parametrize("mode", ["column", "stepwise", "persistent"])
def test_pipeline_built_ring(engine_factory, world, depth, dtype, mode):
    """Steps rotate over `depth` channels (reference pccl/dsl/pipeline.py); consecutive steps of a
    rank are ordered only through the signal chain around the ring."""
    n = world * 4096
    jsons = [compile_to_json_string(pipelined_ring_allreduce(r, world, n, dtype, depth, paired_signals=True))
             for r in range(world)]
    x = seeded_inputs("randn", world, n, dtype, seed=5)
    want = oracle_buffers(jsons, x, dtype)
    # the pipelined schedule computes what the plain ring computes, in the same order
    plain = oracle_buffers(graph_jsons("ring", "build_allreduce", world, n, dtype, "sm", 1), x, dtype)
    assert all(bits_equal(a, b) for a, b in zip(want, plain))
    engine = engine_factory(world)
    got = run(engine, "pipe", jsons, x, mode)
    info = engine.op_info("pipe")
    assert info["residual_signals"] == 0 and info["num_data_ops"] == 2 * (world - 1) * world
    for r in range(world):
        assert bits_equal(got[r], want[r]), f"rank {r}: {mismatch_report(got[r], want[r])}"


def fork_join_graph(rank, chunk, dtype):
    """Per rank, over a tensor of 9 chunks of which the first four are only ever read: four
    independent streams each copy one of the peer's chunks 0..3 into own chunks 4..7; the main
    stream joins all four (one op with four dependencies) and reduces the peer's chunk 0 with own
    chunk 5 into own chunk 4 (read-after-write on stream b, write-after-write on stream a); four
    more streams fork from that op (four successors) and overwrite own chunks 5..8."""
    peer = 1 - rank
    with CommunicationOp(name=f"fj{rank}") as op:
        op.tensor(dtype=dtype, shape=(9 * chunk,))
        for k, name in enumerate("abcd"):
            with Stream(name):
                op.set_channel(k % 2)
                op.sm_copy(source_rank=peer, src_offset=k * chunk, dst_offset=(4 + k) * chunk, size=chunk)
        op.set_channel(0)
        for name in "abcd":
            op.wait(name)
        joined = op.sm_reduce(reduce_op="sum", source_rank=peer, remote_offset=0, src_offset=5 * chunk,
                              dst_offset=4 * chunk, count=chunk)
        for k, name in enumerate("efgh"):
            with Stream(name):
                op.set_channel(1 + k % 2)
                op.wait_for(joined)
                op.sm_copy(source_rank=peer, src_offset=((k + 3) % 4) * chunk, dst_offset=(5 + k) * chunk, size=chunk)
        return op.get_graph()


@pytest.mark.parametrize("mode", ["auto", "stepwise", "persistent"])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_fork_join_over_streams(engine_factory, dtype, mode):
    chunk = 4099          # odd: offsets off 16-byte alignment
    jsons = [compile_to_json_string(fork_join_graph(r, chunk, dtype)) for r in range(2)]
    doc = json.loads(jsons[0])
    assert max(len(o["dependencies"]) for o in doc["operations"]) >= 4
    assert max(len(o["next_ops"]) for o in doc["operations"]) >= 4
    x = seeded_inputs("randn", 2, 9 * chunk, dtype, seed=9)
    want = oracle_buffers(jsons, x, dtype)
    engine = engine_factory(2)
    got = run(engine, "fj", jsons, x, mode)
    info = engine.op_info("fj")
    assert info["position_aligned"] == 0 and info["num_levels"] == 3
    for r in range(2):
        assert bits_equal(got[r], want[r]), f"rank {r}: {mismatch_report(got[r], want[r])}"


@pytest.mark.parametrize("mode", ["stepwise", "persistent", "column"])
def test_noop_nodes_are_contracted(engine_factory, mode):
    """A `noop` between two data ops keeps their order and costs nothing: the linked program has
    the same data ops and levels as the graph without it."""
    world, n = 2, 4096
    base = graph_jsons("ring", "build_allreduce", world, n, "float32", "sm", 1)
    with_noop = []
    for text in base:
        doc = json.loads(text)
        ops = doc["operations"]
        # splice a noop after the first data op: it takes over that op's successors
        k = next(i for i, o in enumerate(ops) if o["primitive"].endswith("reduce"))
        new_index = len(ops)
        noop = {"index": new_index, "executor": "cuda_sm", "primitive": "noop", "channel": ops[k]["channel"],
                "dependencies": [k], "next_ops": list(ops[k]["next_ops"]), "params": {}}
        for nxt in ops[k]["next_ops"]:
            ops[nxt]["dependencies"] = [new_index if d == k else d for d in ops[nxt]["dependencies"]]
        ops[k]["next_ops"] = [new_index]
        ops.append(noop)
        with_noop.append(json.dumps(doc))
    x = seeded_inputs("randn", world, n, "float32", seed=2)
    want = oracle_buffers(base, x, "float32")
    assert all(bits_equal(a, b) for a, b in zip(oracle_buffers(with_noop, x, "float32"), want))
    engine = engine_factory(world)
    got = run(engine, "noop", with_noop, x, mode)
    plain = engine_factory(world)
    for r, j in enumerate(base):
        plain.register_operation_json("plain", j, r)
    a, b = engine.op_info("noop"), plain.op_info("plain")
    assert (a["num_data_ops"], a["num_levels"]) == (b["num_data_ops"], b["num_levels"])
    assert a["num_ops"] == b["num_ops"] + world
    for r in range(world):
        assert bits_equal(got[r], want[r])


@pytest.mark.parametrize("mode", ["auto", "stepwise", "persistent"])
def test_channelized_chain(engine_factory, mode):
    """A chain whose data ops the channelize pass (reference pccl/dsl/passes/channelize.py) has
    moved to other channels while their dependencies still cross those channels: the labels change
    the queues the ops sit in, not their order."""
    from pccl_amd.dsl import Compiler
    world, chunk, pieces = 2, 8192, 8
    jsons = []
    for rank in range(world):
        peer = 1 - rank
        with CommunicationOp(name=f"gather{rank}") as op:
            op.tensor(dtype="float16", shape=(2 * pieces * chunk,))
            for k in range(pieces):     # the peer's first half is never written: no signals needed
                op.sm_copy(source_rank=peer, src_offset=k * chunk, dst_offset=(pieces + k) * chunk, size=chunk)
        jsons.append(Compiler(enable_channelize=True, num_channels=2).compile_to_json(op.get_graph()))
    doc = json.loads(jsons[0])
    assert [o["channel"] for o in doc["operations"]] == [0, 0, 0, 0, 1, 1, 1, 1]
    assert doc["operations"][4]["dependencies"] == [3]          # the chain still crosses the channels
    x = seeded_inputs("randn", world, 2 * pieces * chunk, "float16", seed=11)
    want = oracle_buffers(jsons, x, "float16")
    got = run(engine_factory(world), "chan", jsons, x, mode)
    for r in range(world):
        assert bits_equal(got[r], want[r]), mismatch_report(got[r], want[r])
        assert bits_equal(got[r][pieces * chunk:], x[1 - r][:pieces * chunk])


@pytest.mark.parametrize("alg,world,n,dtype", [("ring", 8, 1 << 16, "bfloat16"), ("tree", 8, 5000, "float32")])
def test_level_runner_graph_replays(engine_factory, alg, world, n, dtype):
    """The level runner captures the launches of one execution as a HIP graph per set of rank
    pointers.  Every replay - with other GPU work and synchronisations of the program in between,
    on fresh data in the same tensors, and on a second set of tensors - must give what launching
    level by level gives."""
    jsons = graph_jsons(alg, "build_allreduce", world, n, dtype, "sm", 1)
    engine = engine_factory(world)
    for r, j in enumerate(jsons):
        engine.register_operation_json("g", j, r)
    engine.set_option("mode", "stepwise")
    sets = [[torch.empty(n, dtype=seeded_inputs("randn", 1, 1, dtype)[0].dtype, device="cuda") for _ in range(world)]
            for _ in range(2)]
    scratch = torch.zeros(1 << 20, device="cuda")
    for rep in range(6):
        x = seeded_inputs("randn", world, n, dtype, seed=100 + rep)
        want = oracle_buffers(jsons, x, dtype)
        bufs = sets[rep % 2]
        engine.set_option("level_graph", 0 if rep == 4 else 1)      # one eager execution in the middle
        for b, t in zip(bufs, x):
            b.copy_(t)
        scratch.add_(1.0)                        # unrelated eager work on the same stream
        engine.execute_inplace("g", bufs)
        total = scratch.sum()                    # a library reduction between the replays
        torch.cuda.synchronize()
        assert total.item() == (rep + 1) * (1 << 20)
        for r in range(world):
            assert bits_equal(bufs[r], want[r]), f"replay {rep}, rank {r}: {mismatch_report(bufs[r], want[r])}"
    engine.set_option("level_graph", 1)
    # staged calls in this mode go through the engine's rank buffers: one more pointer set
    x = seeded_inputs("randn", world, n, dtype, seed=55)
    want = oracle_buffers(jsons, x, dtype)
    for _ in range(2):
        outs = engine.execute_operation("g", [t.cuda() for t in x])
        for r in range(world):
            assert bits_equal(outs[r], want[r])
    engine.set_option("level_graph", 0)
