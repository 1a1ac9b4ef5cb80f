"""Schedule emitter: byte-for-byte agreement with graphs captured from the reference's own emitter,
and the structural expectations the reference's unit tests state.

tests/golden/graphs/*.json were produced by tests/golden/make_graph_fixtures.py, which drives the
reference's schedule templates, passes and JSON generator (read-only, in the authoring container).
"""
import json
import os

import pytest

from helpers import GOLDEN
from helpers import chained_gather, pipelined_ring_allreduce
from pccl_amd.dsl.channelize import (H100_PROFILE, MI355X_PROFILE, ChannelizePass, DeviceProfile,
                                     critical_path_cost_us, op_latency_us)
from pccl_amd.dsl import (ALGORITHMS, CommunicationOp, Compiler, Pipeline, RecursiveHalvingDoubling, RingAllreduce,
                          Stream, TreeAllreduce, build_graph, compile_to_json_string, ragged_cuts)

with open(os.path.join(GOLDEN, "graphs", "index.json")) as f:
    INDEX = json.load(f)


@pytest.mark.parametrize("case", INDEX, ids=[c["stem"] for c in INDEX])
def test_emitted_json_equals_reference_emitter(case):
    for rank in range(case["world_size"]):
        if case["algorithm"] == "pipelined_ring":    # built with the Pipeline construct (reference pipeline.py)
            g = pipelined_ring_allreduce(rank, case["world_size"], case["tensor_size"], case["dtype"],
                                         case["num_channels"])
        elif case["algorithm"] == "chained_gather":  # compiled with the channelize pass switched on
            g = chained_gather(rank, case["world_size"], case["tensor_size"] // case["pieces"], case["dtype"],
                               case["pieces"], case["method"])
            mine = Compiler(enable_channelize=True, num_channels=case["num_channels"]).compile_to_dict(g)
            with open(os.path.join(GOLDEN, "graphs", f"{case['stem']}_rank{rank}.json")) as f:
                assert json.dumps(mine) == json.dumps(json.load(f)), f"rank {rank}"
            continue
        else:
            g = getattr(ALGORITHMS[case["algorithm"]](), case["method"])(
                rank, case["world_size"], case["tensor_size"], dtype=case["dtype"],
                executor=case["executor"], num_channels=case["num_channels"])
        mine = json.loads(compile_to_json_string(g))
        with open(os.path.join(GOLDEN, "graphs", f"{case['stem']}_rank{rank}.json")) as f:
            ref = json.load(f)
        # same keys in the same order, same values: compare the canonical re-serialisation
        assert json.dumps(mine) == json.dumps(ref), f"rank {rank}"


# --- structural expectations (reference tests/test_algorithms.py) ------------------------------

def test_ring_8_ranks_has_44_ops():          # tests/test_algorithms.py:31-33
    assert RingAllreduce().build_allreduce(rank=0, world_size=8, tensor_size=8192).size() == 44


def test_ring_grows_with_world_size():       # :38-43
    sizes = [RingAllreduce().build_allreduce(0, w, 1024 * w).size() for w in (2, 4, 8)]
    assert sizes[0] < sizes[1] < sizes[2]


def test_ring_multichannel_uses_both_channels():   # :45-50
    g1 = RingAllreduce().build_allreduce(0, 2, 2048, num_channels=1)
    g2 = RingAllreduce().build_allreduce(0, 2, 2048, num_channels=2)
    assert g2.size() > g1.size()
    assert {o.channel for o in g2.ops.values()} == {0, 1}


def test_ring_sm_executor_emits_sm_primitives():   # :52-56
    g = RingAllreduce().build_allreduce(0, 2, 2048, executor="sm")
    assert any(o.primitive in ("sm.copy", "sm.reduce") for o in g.ops.values())
    g = RingAllreduce().build_allreduce(0, 2, 2048)      # the templates default to "tma"
    assert any(o.primitive in ("tma.copy", "tma.reduce") for o in g.ops.values())


def test_rhd_fewer_ops_than_ring_at_8():     # :76-79
    assert (RecursiveHalvingDoubling().build_allreduce(0, 8, 8192).size()
            < RingAllreduce().build_allreduce(0, 8, 8192).size())


@pytest.mark.parametrize("cls", [RecursiveHalvingDoubling, TreeAllreduce])
def test_power_of_two_is_required(cls):      # :84-86, :121-123
    with pytest.raises(ValueError, match="power-of-2"):
        cls().build_allreduce(rank=0, world_size=3, tensor_size=3072)


def test_rhd_partner_pattern():              # :91-98
    g = RecursiveHalvingDoubling().build_allreduce(rank=0, world_size=4, tensor_size=4096)
    partners = {o.params["target_rank"] for o in g.ops.values() if o.primitive == "notify"}
    assert partners == {1, 2}


def test_tree_root_reduces_the_whole_tensor():     # :128-132
    g = TreeAllreduce().build_allreduce(rank=0, world_size=4, tensor_size=4096)
    reduces = [o for o in g.ops.values() if o.primitive.endswith(".reduce")]
    assert reduces and all(o.params["count"] == 4096 for o in reduces)


def test_algorithm_properties():
    assert RingAllreduce().name == "ring" and RingAllreduce().bandwidth_optimal
    assert RingAllreduce().step_count == "O(2(N-1))"
    assert RecursiveHalvingDoubling().name == "rhd" and RecursiveHalvingDoubling().step_count == "O(2 log N)"
    assert TreeAllreduce().name == "tree" and not TreeAllreduce().bandwidth_optimal
    assert set(ALGORITHMS) == {"ring", "rhd", "tree"}


# --- JSON v2 document (reference tests/test_basic.py:454-464,561-570; test_multichannel.py:99-113) --

def test_document_has_the_v2_fields():
    doc = json.loads(compile_to_json_string(RingAllreduce().build_allreduce(1, 4, 4096, num_channels=2)))
    assert doc["version"] == 2
    assert doc["tensor_info"] == {"dtype": "bfloat16", "shape": [4096]}
    assert doc["collective_type"] == "allreduce"
    assert doc["executors"] == ["cuda_sm", "cuda_tma"]
    for i, op in enumerate(doc["operations"]):
        assert op["index"] == i
        assert set(op) == {"index", "executor", "primitive", "channel", "dependencies", "next_ops", "params"}
        for d in op["dependencies"]:
            assert d < i                      # indices are a topological order
    assert {op["channel"] for op in doc["operations"]} == {0, 1}


def test_builder_chains_per_stream_and_joins_on_wait():
    with CommunicationOp(name="t") as op:
        op.tensor(dtype="float32", shape=(64,))
        with Stream("a"):
            a1 = op.sm_copy(source_rank=1, src_offset=0, dst_offset=0, size=32)
            a2 = op.notify(signal_id=1, target_rank=1)
        with Stream("b"):
            b1 = op.sm_copy(source_rank=1, src_offset=32, dst_offset=32, size=32)
            op.wait("a")
            b2 = op.notify(signal_id=2, target_rank=1)
    g = op.get_graph()
    assert a2.deps == [a1.uid] and b1.deps == []
    assert set(b2.deps) == {a2.uid, b1.uid}
    doc = Compiler().compile_to_dict(g)
    assert len(doc["operations"]) == 4


def test_invalid_arguments_are_rejected():
    with pytest.raises(ValueError, match="unsupported dtype"):
        with CommunicationOp(name="t") as op:
            op.tensor(dtype="float64", shape=(4,))
    with pytest.raises(ValueError, match="shape must be a tuple"):
        with CommunicationOp(name="t") as op:
            op.tensor(dtype="float32", shape=[4])
    with pytest.raises(ValueError, match="invalid reduce_op"):
        build_graph("t", lambda op: (op.tensor("float32", (4,)),
                                     op.sm_reduce(source_rank=0, src_offset=0, dst_offset=0, remote_offset=0,
                                                  count=4, reduce_op="prod")))
    with pytest.raises(ValueError, match="source_rank"):
        build_graph("t", lambda op: (op.tensor("float32", (4,)),
                                     op.sm_copy(source_rank=-1, src_offset=0, dst_offset=0, size=4)))
    with pytest.raises(RuntimeError, match="within a CommunicationOp"):
        with Stream("x"):
            pass
    with pytest.raises(ValueError, match="empty"):
        Compiler().compile(CommunicationOp(name="e").get_graph())


def test_ragged_cuts_rule():
    cuts = ragged_cuts(25_165_824, 8, seed=0)
    assert len(cuts) == 7 and cuts == sorted(cuts)
    assert all(c % 4 in (1, 2, 3) for c in cuts)          # never on a 16-byte boundary for 4-byte types
    assert ragged_cuts(25_165_824, 8, seed=0) == cuts      # deterministic
    g = TreeAllreduce().build_allreduce(0, 4, 4099, dtype="int32", executor="sm", cuts=ragged_cuts(4099, 5))
    reduces = [o for o in g.ops.values() if o.primitive == "sm.reduce"]
    assert sum(o.params["count"] for o in reduces) == 2 * 4099   # rank 0 reduces twice over the whole tensor


def test_pipeline_construct():                # reference pccl/dsl/pipeline.py:64-88
    with pytest.raises(ValueError):
        Pipeline(depth=0)
    with CommunicationOp(name="p") as op:
        op.tensor(dtype="float32", shape=(64,))
        pipe = Pipeline(depth=2)
        with pytest.raises(RuntimeError):
            with pipe.stage():
                pass
        with pipe.bind(op):
            made = []
            for k in range(5):
                with pipe.stage():
                    made.append(op.sm_copy(source_rank=1, src_offset=0, dst_offset=0, size=8))
    doc = json.loads(compile_to_json_string(op.get_graph()))
    ops = sorted(doc["operations"], key=lambda o: o["index"])
    assert sorted(o["channel"] for o in ops) == [0, 0, 0, 1, 1]
    # stages of one channel are chained, channels are independent: two roots, two leaves
    assert sum(1 for o in ops if not o["dependencies"]) == 2
    assert sum(1 for o in ops if not o["next_ops"]) == 2
    for o in ops:
        for d in o["dependencies"]:
            assert ops[d]["channel"] == o["channel"]


def test_cost_model_closed_forms():            # reference pccl/dsl/superopt/cost_model.py:113-200
    p = H100_PROFILE
    assert op_latency_us("notify", p) == 1.0
    assert op_latency_us("sm.copy", p, 50_000) == pytest.approx(1.0 + 1.0)           # 50 KB at 50 GB/s
    # reduce: max(transfer, compute): 120,000 B at 60 GB/s = 2 us; 30,000 elements at 35 Gop/s = 0.857 us
    assert op_latency_us("tma.reduce", p, 120_000) == pytest.approx(1.0 + 2.0)
    chain = [("sm.copy", 0)] * 4
    edges = [(0, 1), (1, 2), (2, 3)]
    assert critical_path_cost_us(chain, edges, p, 50_000) == pytest.approx(8.0)
    split = [("sm.copy", 0), ("sm.copy", 0), ("sm.copy", 1), ("sm.copy", 1)]
    assert critical_path_cost_us(split, [(0, 1), (2, 3)], p, 50_000) == pytest.approx(4.0 + 0.5)
    assert critical_path_cost_us([], [], p) == 0.0
    q = DeviceProfile.from_dict(MI355X_PROFILE.to_dict())
    assert q == MI355X_PROFILE and q.bandwidth_gb_s["tma"] == q.bandwidth_gb_s["sm"]


def test_channelize_leaves_non_contiguous_chains_alone():
    """The ring template's consecutive steps work on descending chunks, which do not follow one
    another, so the pass changes nothing there (whatever the profile)."""
    for profile in (H100_PROFILE, MI355X_PROFILE):
        g = RingAllreduce().build_allreduce(0, 8, 8 * 65536, dtype="float32", executor="sm")
        before = json.dumps(Compiler().compile_to_dict(g))
        g2 = RingAllreduce().build_allreduce(0, 8, 8 * 65536, dtype="float32", executor="sm")
        after = json.dumps(Compiler(enable_channelize=True, num_channels=2, device_profile=profile).compile_to_dict(g2))
        assert before == after
    g = chained_gather(0, 2, 65536, "float32", 8, "copy")
    ChannelizePass(num_channels=4, profile=MI355X_PROFILE).run(g)
    assert sorted({o.channel for o in g.ops.values() if o.is_data}) == [0, 1, 2, 3]


def test_algorithm_selector():                 # reference pccl/dsl/algorithms/selector.py:24-56
    from pccl_amd.dsl.algorithms import select_algorithm, select_algorithm_cost_based
    from pccl_amd.dsl.algorithms.selector import graph_cost_us
    MB = 1 << 20
    table = {(8, 4 * MB): RingAllreduce, (8, MB): RingAllreduce, (8, MB - 1): RecursiveHalvingDoubling,
             (4, 1024): RecursiveHalvingDoubling, (2, 1024): RingAllreduce, (6, 1024): RingAllreduce,
             (3, 64 * MB): RingAllreduce, (16, 65536): RecursiveHalvingDoubling}
    for (world, size), want in table.items():
        assert type(select_algorithm(world, size)) is want, (world, size)
    # cost based: the candidate with the smallest critical path, found independently here
    for world, nbytes, profile in ((8, 4096, H100_PROFILE), (8, 64 * MB, H100_PROFILE), (16, 4096, MI355X_PROFILE),
                                   (6, 4096, H100_PROFILE)):
        cands = [RingAllreduce()] + ([RecursiveHalvingDoubling(), TreeAllreduce()] if world & (world - 1) == 0 else [])
        costs = [graph_cost_us(a.build_allreduce(rank=1, world_size=world, tensor_size=world * 1024,
                                                 dtype="bfloat16", executor="tma"), profile, nbytes) for a in cands]
        got = select_algorithm_cost_based(1, world, world * 1024, nbytes, device=profile)
        assert type(got) is type(cands[costs.index(min(costs))])
    # log-step schedules have the shorter critical path for small messages on 8 ranks
    assert type(select_algorithm_cost_based(0, 8, 8192, 1024)) is not RingAllreduce


def test_superopt_upgrades_sm_to_tma():        # reference tests/test_superopt.py:813-851
    """The executor upgrades of the reference's superoptimisation pass: no cuda_sm data executor is
    left, the document keeps its fields, and the result is the document the tma template gives."""
    from pccl_amd.dsl import Compiler
    world, n = 4, 4096
    for r in range(world):
        sm = RingAllreduce().build_allreduce(r, world, n, dtype="bfloat16", executor="sm", num_channels=2)
        tma = RingAllreduce().build_allreduce(r, world, n, dtype="bfloat16", executor="tma", num_channels=2)
        doc = Compiler(enable_superopt=True, topology=None).compile_to_dict(sm)
        assert doc["version"] == 2 and doc["operations"]
        data = {op["executor"] for op in doc["operations"] if op["primitive"] not in ("notify", "wait_notify", "noop")}
        assert data == {"cuda_tma"}
        required = {"index", "executor", "primitive", "channel", "dependencies", "next_ops", "params"}
        assert all(required <= set(op) for op in doc["operations"])
        assert doc == Compiler().compile_to_dict(tma)
    plain = Compiler().compile_to_dict(RingAllreduce().build_allreduce(0, world, n, dtype="bfloat16", executor="sm"))
    assert {op["executor"] for op in plain["operations"]} == {"cuda_sm"}
