"""The column planner on the CPU: the programs it emits, executed here by two small interpreters
(values re-read through memory / values kept in per-rank slots with only the last value of a rank
written out), must reproduce the oracle's buffers.  int32 keeps the interpreters trivially exact;
the instruction semantics do not depend on the dtype.

What this pins without a GPU: segment cutting, accumulator forwarding, dead-store elimination,
last-write marking, first-touch lists, the broadcast tail, and the windows / dropped stores /
pass-through copies of staged calls that run on the caller's tensors.
"""
import json

import numpy as np
import pytest

from helpers import graph_jsons, oracle, pipelined_ring_allreduce, random_program
from pccl_amd._lib import HostGraph, HostProgram
from pccl_amd.dsl import compile_to_json_string, ragged_cuts

GARBAGE = np.int32(-0x5A5A5A5B)


def red(op, a, b):
    if op == 0:
        return (a.astype(np.int64) + b.astype(np.int64)).astype(np.int32)   # wraps like the device
    return np.maximum(a, b) if op == 1 else np.minimum(a, b)


def fields(word):
    return [(word >> (8 * i)) & 0xFF for i in range(8)]


def run_plan(plan, first_src, mem, slots_mode):
    """Execute every segment.  `first_src[r]` is where a first touch of rank r reads, `mem[r]` where
    stores and re-reads go (the same arrays for in-place execution)."""
    for seg in plan["segments"]:
        lo, hi = seg.start, seg.end
        prog = plan["instrs"][seg.prog_start:seg.prog_start + seg.prog_len]
        assert seg.prog_start % 4 == 0 and seg.prog_len % 4 == 0       # four instructions per scalar load
        slot = {}
        if slots_mode:
            listed = []
            for w in plan["pre"][seg.pre_start:seg.pre_start + seg.pre_words]:
                listed += [b for b in fields(w) if b != 0xFF]
            assert len(set(listed)) == len(listed)
            for r in listed:
                slot[r] = first_src[r][lo:hi].copy()
        acc = np.zeros(hi - lo, np.int32)
        for w in prog:
            self_, peer, a_src, b_src, op, store, a_first, b_first = fields(w)
            kind, last = store & 3, bool(store & 4)

            def operand(src, rank, first):
                if src == 2:
                    return acc
                if slots_mode:
                    return slot[rank]               # KeyError = a value the plan never put on chip
                return (first_src if first else mem)[rank][lo:hi]
            a = operand(a_src, peer, a_first)
            acc = red(op, a, operand(b_src, self_, b_first)) if b_src else a.copy()
            if slots_mode:
                if kind == 1:
                    slot[self_] = acc.copy()
                if kind == 2 or (kind == 1 and last):
                    mem[self_][lo:hi] = acc
            elif kind:
                mem[self_][lo:hi] = acc
        for r in range(64):
            if seg.bcast_mask >> r & 1:
                mem[r][lo:hi] = acc


def inputs_for(world, n, seed):
    rng = np.random.default_rng(seed)
    return [rng.integers(-1000, 1000, n, dtype=np.int32) for _ in range(world)]


def link(jsons):
    return HostProgram([HostGraph.from_json(j) for j in jsons])


ALLREDUCE = [
    ("ring", 3, 3 * 64, 1, {}), ("ring", 4, 4096, 2, {}), ("ring", 8, 8 * 96, 4, {}),
    ("rhd", 8, 1024, 1, {}), ("rhd", 16, 16 * 40, 2, {}), ("tree", 8, 777, 1, {}), ("tree", 32, 4100, 1, {}),
    ("tree", 16, 5000, 1, {"cuts": "ragged", "reduce_op": "max"}), ("ring", 4, 4 * 50, 1, {"reduce_op": "min"}),
]


@pytest.mark.parametrize("alg,world,n,channels,ext", ALLREDUCE)
@pytest.mark.parametrize("slots_mode", [False, True], ids=["memory", "slots"])
def test_in_place_plan_reproduces_the_oracle(alg, world, n, channels, ext, slots_mode):
    ext = dict(ext)
    if ext.get("cuts") == "ragged":
        ext["cuts"] = ragged_cuts(n, 5, seed=1)
    jsons = graph_jsons(alg, "build_allreduce", world, n, "int32", "sm", channels, **ext)
    x = inputs_for(world, n, 3)
    want = [a.copy() for a in x]
    oracle.run([oracle.Graph(json.loads(j)) for j in jsons], want)
    prog = link(jsons)
    plan = prog.column_plan()
    assert prog.info()["position_aligned"] == 1 and plan["segments"]
    bufs = [a.copy() for a in x]
    run_plan(plan, bufs, bufs, slots_mode)
    for r in range(world):
        assert np.array_equal(bufs[r], want[r]), f"rank {r}"
    # allreduce programs end in a broadcast: some segment must have used the mask
    assert any(s.bcast_mask for s in plan["segments"])


@pytest.mark.parametrize("depth", [2, 3])
@pytest.mark.parametrize("slots_mode", [False, True], ids=["memory", "slots"])
def test_pipelined_ring_plan(depth, slots_mode):
    world, n = 4, 4 * 128
    jsons = [compile_to_json_string(pipelined_ring_allreduce(r, world, n, "int32", depth, paired_signals=True))
             for r in range(world)]
    x = inputs_for(world, n, 5)
    want = [a.copy() for a in x]
    oracle.run([oracle.Graph(json.loads(j)) for j in jsons], want)
    bufs = [a.copy() for a in x]
    run_plan(link(jsons).column_plan(), bufs, bufs, slots_mode)
    assert all(np.array_equal(b, w) for b, w in zip(bufs, want))


@pytest.mark.parametrize("method", ["build_allreduce", "build_reduce_scatter", "build_allgather"])
@pytest.mark.parametrize("world,channels", [(4, 1), (8, 1), (8, 2)])
@pytest.mark.parametrize("slots_mode", [False, True], ids=["memory", "slots"])
def test_staged_plan_reads_inputs_and_writes_outputs_only(method, world, channels, slots_mode):
    """Staged semantics (reference engine_c.cc:468-548): input r goes into buffer r at its window,
    the program runs, the output window of buffer r comes back.  The staged plan must produce
    exactly those windows while reading nothing but the input windows (everything else is poisoned
    here) and leaving everything outside the output windows untouched."""
    n = world * 96
    jsons = graph_jsons("ring", method, world, n, "int32", "tma", channels)
    prog = link(jsons)
    plan = prog.column_plan(staged=True)
    if not plan["segments"]:
        # two-channel allgather gathers pieces that lie outside the staged chunk: no staged plan, the
        # library stages through its rank buffers instead
        assert method == "build_allgather" and channels == 2
        return
    rng = np.random.default_rng(7)
    bufs, ins, outs = [], [], []
    for r in range(world):
        (i0, i1), (o0, o1) = plan["in_window"][r], plan["out_window"][r]
        full_in = np.full(n, GARBAGE, np.int32)
        full_in[i0:i1] = rng.integers(-1000, 1000, i1 - i0, dtype=np.int32)
        buf = np.zeros(n, np.int32)
        buf[i0:i1] = full_in[i0:i1]
        bufs.append(buf); ins.append(full_in); outs.append(np.full(n, GARBAGE, np.int32))
    oracle.run([oracle.Graph(json.loads(j)) for j in jsons], bufs)
    run_plan(plan, ins, outs, slots_mode)
    for r in range(world):
        o0, o1 = plan["out_window"][r]
        assert np.array_equal(outs[r][o0:o1], bufs[r][o0:o1]), f"rank {r}"
        assert np.all(outs[r][:o0] == GARBAGE) and np.all(outs[r][o1:] == GARBAGE)
    info = prog.info()
    S = n * 4
    if method != "build_allreduce" and channels == 1:
        assert info["staged_load_bytes"] + info["staged_store_bytes"] == (world + 1) * S   # R S one way, S the other


@pytest.mark.parametrize("seed", range(12))
@pytest.mark.parametrize("slots_mode", [False, True], ids=["memory", "slots"])
def test_random_aligned_programs(seed, slots_mode):
    """Random race-free programs (random ranks, peers, ranges of any parity, sum / max / min) whose ops
    read and write the same positions: segments of many different op lists, forwarding, dead stores
    and re-reads in every combination."""
    world, n = 2 + seed % 5, 600 + 37 * seed
    jsons = random_program(seed, world, n, 30 + 5 * seed, "int32", aligned=True, reduce_ops=("sum", "max", "min"))
    x = inputs_for(world, n, seed)
    want = [a.copy() for a in x]
    oracle.run([oracle.Graph(json.loads(j)) for j in jsons], want)
    prog = link(jsons)
    assert prog.info()["position_aligned"] == 1
    bufs = [a.copy() for a in x]
    run_plan(prog.column_plan(), bufs, bufs, slots_mode)
    for r in range(world):
        assert np.array_equal(bufs[r], want[r]), f"rank {r}"


# ---------------------------------------------------------------------------------------------
# Chain form of the plans (what the phased runner executes)

def _info(alg, method, world, n, dtype, channels=1, **ext):
    graphs = [HostGraph.from_json(j) for j in graph_jsons(alg, method, world, n, dtype, "sm", channels, **ext)]
    return HostProgram(graphs).info()


def test_which_plans_are_chains():
    """A plan is a chain plan when every segment leaves one value - every contributing rank combined
    once - in all the ranks it writes: ring allreduces literally; trees and halving-doubling when the
    operator may be re-associated for the element type (integer sums, maxima, minima), else as
    balanced trees; a staged reduce_scatter but not the in-place one, which leaves its partial sums
    in the other ranks."""
    ring = _info("ring", "build_allreduce", 8, 1 << 16, "bfloat16", 4)
    assert ring["chain_segments"] == ring["num_segments"] == 32 and ring["staged_chain_segments"] == 32
    rs = _info("ring", "build_reduce_scatter", 8, 1 << 16, "float16")
    assert rs["chain_segments"] == 0 and rs["staged_chain_segments"] == 8
    ag = _info("ring", "build_allgather", 8, 1 << 16, "float16")
    assert ag["chain_segments"] == 8 and ag["staged_chain_segments"] == 8
    for dtype, op in (("int32", "sum"), ("float32", "max"), ("bfloat16", "min"), ("float32", "sum"), ("float16", "sum")):
        tree = _info("tree", "build_allreduce", 32, 1 << 12, dtype, reduce_op=op)
        assert tree["chain_segments"] == tree["num_segments"] == 1, (dtype, op)
    rhd = _info("rhd", "build_allreduce", 16, 1 << 16, "float32", 2)
    assert rhd["chain_segments"] == rhd["num_segments"]
    # a reduce-only ring (no allgather phase) leaves a different value in every rank
    with_partials = random_program(77, 4, 5000, 30, "int32", True)
    assert HostProgram([HostGraph.from_json(j) for j in with_partials]).info()["chain_segments"] == 0
