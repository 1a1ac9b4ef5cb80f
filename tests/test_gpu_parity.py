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
    ("ring", 8, 1 << 16, "float8_e4m3", 2, "randn"),       # fp8: add in f16, saturating narrow
    ("rhd", 8, 1 << 15, "float8_e5m2", 1, "randn"),
    ("ring", 24, 24 * 2731, "bfloat16", 1, "randn"),       # more than 16 ranks and nothing read back:
                                                           # column mode picks the register runner
]


MODES = ["column", "stepwise", "persistent"]


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


@pytest.mark.parametrize("fuse", [1, 0])
@pytest.mark.parametrize("channels", [1, 2])
@pytest.mark.parametrize("mode", MODES)
def test_reduce_scatter_and_allgather(engine_factory, mode, channels, fuse):
    """reference tests/test_correctness.py:196-241: reduce_scatter output is one chunk of sums;
    allgather input is one chunk, output the concatenation.  With two channels the reduced pieces
    of a rank are not contiguous; the output is still "chunk r of buffer r" as the reference's
    engine defines it.  fuse=1 runs on the caller's tensors, fuse=0 through the rank buffers."""
    world, n = 8, 1 << 16
    chunk = n // world
    engine = engine_factory(world)
    engine.set_option("fuse_staging", fuse)
    try:
        jsons = graph_jsons("ring", "build_reduce_scatter", world, n, "float16", "tma", channels)
        inputs = seeded_inputs("randn0.1", world, n, "float16")
        expect = oracle_buffers(jsons, inputs, "float16")
        got, _ = run_gpu(engine, jsons, inputs, mode, out_elems=chunk)
        for r in range(world):
            assert bits_equal(got[r], expect[r][r * chunk:(r + 1) * chunk]), mismatch_report(got[r], expect[r][r * chunk:(r + 1) * chunk])

        jsons = graph_jsons("ring", "build_allgather", world, n, "float16", "tma", channels)
        parts = seeded_inputs("randn0.1", world, chunk, "float16", seed=1)
        expect = oracle_buffers(jsons, parts, "float16", place=lambda r: r * chunk, buffer_elems=n)
        got, _ = run_gpu(engine, jsons, parts, mode, out_elems=n)
        for r in range(world):
            if channels == 1:
                assert bits_equal(got[r], torch.cat(parts)), f"rank {r}"
            else:
                # with two channels the graph gathers, per channel, piece q from rank q; only where
                # that piece lies inside the chunk rank q staged is its content defined by the
                # inputs (elsewhere it is whatever the rank buffer held), so compare those pieces
                per_ch, per_rank = n // channels, n // channels // world
                for c in range(channels):
                    for q in range(world):
                        lo = c * per_ch + q * per_rank
                        src_lo = q * chunk
                        if src_lo <= lo and lo + per_rank <= src_lo + chunk:
                            assert bits_equal(got[r][lo:lo + per_rank], expect[r][lo:lo + per_rank])
    finally:
        engine.set_option("fuse_staging", 1)


@pytest.mark.parametrize("mode", ["auto", "stepwise", "persistent"])
@pytest.mark.parametrize("world,n", [(4, 1 << 12), (8, 8 * 1031), (3, 3 * 5000)])
def test_alltoall(engine_factory, mode, world, n):
    """reference tests/test_correctness.py:243-272: out[i] chunk = chunk r of rank i's input.  In
    `auto` mode the staged call is composed into direct input-to-output copies (one launch); the
    other modes stage through the rank buffers and their scratch region."""
    chunk = n // world
    jsons = graph_jsons("ring", "build_alltoall", world, n, "bfloat16", "tma", 1)
    inputs = seeded_inputs("randn", world, n, "bfloat16", seed=13)
    got, info = run_gpu(engine_factory(world), jsons, inputs, mode)
    assert info["position_aligned"] == 0 and info["num_gather_copies"] == world * world
    for r in range(world):
        want = torch.cat([inputs[i][r * chunk:(r + 1) * chunk] for i in range(world)])
        assert bits_equal(got[r], want), mismatch_report(got[r], want)


def test_alltoall_falls_back_to_staging_when_it_must(engine_factory):
    """Outputs that overlap inputs, or fuse_staging=0: the same result through the rank buffers."""
    world, n = 4, 1 << 13
    chunk = n // world
    jsons = graph_jsons("ring", "build_alltoall", world, n, "float32", "sm", 1)
    engine = engine_factory(world)
    for r, j in enumerate(jsons):
        engine.register_operation_json("a2a", j, r)
    x = seeded_inputs("randn", world, n, "float32", seed=3)
    want = [torch.cat([x[i][r * chunk:(r + 1) * chunk] for i in range(world)]) for r in range(world)]
    dev = [t.cuda() for t in x]
    outs = engine.execute_operation("a2a", dev, dev)          # in place: every output is an input
    for r in range(world):
        assert bits_equal(outs[r], want[r])
    engine.set_option("fuse_staging", 0)
    outs = engine.execute_operation("a2a", [t.cuda() for t in x])
    engine.set_option("fuse_staging", 1)
    for r in range(world):
        assert bits_equal(outs[r], want[r])


def test_persistent_runner_reports_a_wait_that_expires(engine_factory):
    """Every wait of the persistent runner is bounded.  With the bound set to zero the first
    workgroup that finds a predecessor not yet published gives up at once: it records which, every
    other wait ends as soon as it sees that record, the launch drains normally, and the call reports
    the stall instead of hanging.  The next execution, with the bound restored, is correct."""
    from pccl_amd._lib import PcclError
    world, n = 8, 1 << 24
    jsons = graph_jsons("ring", "build_allreduce", world, n, "float32", "sm", 1)
    engine = engine_factory(world)
    for r, j in enumerate(jsons):
        engine.register_operation_json("slow", j, r)
    engine.set_option("mode", "persistent")
    engine.set_option("wait_timeout_ms", 0)
    bufs = [torch.ones(n, device="cuda") for _ in range(world)]
    with pytest.raises(PcclError, match="gave up waiting"):
        engine.execute_inplace("slow", bufs, sync=True)
    engine.set_option("wait_timeout_ms", 2000)
    for b in bufs:
        b.fill_(1.0)
    engine.execute_inplace("slow", bufs, sync=True)
    assert all(torch.all(b == world) for b in bufs)
    engine.set_option("mode", "auto")


# ---------------------------------------------------------------------------------------------
# Staged calls: fused into the program (default) and through the engine's rank buffers.

def _ring_partial(kind, rank, world, n):
    """The reference's reduce-only / copy-only ring graphs (tests/test_correctness.py:46-90):
    no collective_type, so the engine stages them like an allreduce."""
    from pccl_amd.dsl import CommunicationOp, compile_to_json_string
    chunk = n // world
    prev, nxt = (rank - 1) % world, (rank + 1) % world
    with CommunicationOp(name=f"test_{kind}_rank{rank}") as op:
        op.tensor(dtype="bfloat16", shape=(n,))
        op.notify(signal_id=100, target_rank=nxt)
        op.wait_notify(signal_id=100, source_rank=prev)
        for step in range(world - 1):
            c = (rank - step - 1) % world if kind == "reduce" else (rank - step) % world
            if step > 0:
                op.wait_notify(signal_id=0, source_rank=prev)
            if kind == "reduce":
                op.tma_reduce(reduce_op="sum", source_rank=prev, src_offset=c * chunk, dst_offset=c * chunk,
                              remote_offset=c * chunk, count=chunk)
            else:
                op.tma_copy(source_rank=prev, src_offset=c * chunk, dst_offset=c * chunk, size=chunk)
            op.notify(signal_id=0, target_rank=nxt)
        op.wait_notify(signal_id=0, source_rank=prev)
    return compile_to_json_string(op.get_graph())


@pytest.mark.parametrize("mode", ["auto", "column", "stepwise", "persistent"])
@pytest.mark.parametrize("what", ["no operations", "zero-size data ops"])
def test_empty_graphs_and_zero_size_ops_leave_the_data_alone(engine_factory, what, mode):
    """A graph without operations, and a ring whose reduces and copies all have size 0 (its notify /
    wait chain intact), register and run; nothing is moved.  In the reference's call shape the input
    is staged into the rank buffer and the output read back from it (engine_c.cc:524-543), so the
    output equals the input; in place the buffers keep their contents.  The oracle agrees."""
    import json
    world, n = 4, 4096
    docs = [json.loads(t) for t in graph_jsons("ring", "build_allreduce", world, n, "float32", "sm", 1)]
    for d in docs:
        if what == "no operations":
            d["operations"] = []
        else:
            for op in d["operations"]:
                for key in ("size", "count"):
                    if key in op.get("params", {}):
                        op["params"][key] = 0
    jsons = [json.dumps(d) for d in docs]
    inputs = seeded_inputs("randn", world, n, "float32", seed=11)
    expect = oracle_buffers(jsons, inputs, "float32")
    for r in range(world):
        assert bits_equal(expect[r], inputs[r])
    engine = engine_factory(world)
    got, info = run_gpu(engine, jsons, inputs, mode, inplace=True)
    assert info["algorithmic_bytes"] == 0
    for r in range(world):
        assert bits_equal(got[r], inputs[r]), f"in place, rank {r}"
    got, _ = run_gpu(engine, jsons, inputs, mode)
    for r in range(world):
        assert bits_equal(got[r], inputs[r]), f"staged, rank {r}"
    engine.set_option("mode", "auto")


@pytest.mark.parametrize("fuse", [1, 0])
@pytest.mark.parametrize("kind", ["reduce", "copy"])
def test_partial_ring_graphs_pass_untouched_chunks_through(engine_factory, kind, fuse):
    """Chunks a graph never writes must come out as they went in, whichever way the call is staged
    (closed forms of reference tests/test_correctness.py:150-161,180-189)."""
    world, n = 4, 1 << 14
    jsons = [_ring_partial(kind, r, world, n) for r in range(world)]
    inputs = seeded_inputs("randn", world, n, "bfloat16", seed=3)
    expect = oracle_buffers(jsons, inputs, "bfloat16")
    engine = engine_factory(world)
    engine.set_option("fuse_staging", fuse)
    try:
        got, info = run_gpu(engine, jsons, inputs, "column")
    finally:
        engine.set_option("fuse_staging", 1)
    for r in range(world):
        assert bits_equal(got[r], expect[r]), f"rank {r}: {mismatch_report(got[r], expect[r])}"


@pytest.mark.parametrize("fuse", [1, 0])
def test_staged_call_with_output_aliasing_input(engine_factory, fuse):
    world, n = 8, 1 << 15
    jsons = graph_jsons("ring", "build_allreduce", world, n, "float32", "sm", 2)
    inputs = seeded_inputs("randn", world, n, "float32", seed=5)
    expect = oracle_buffers(jsons, inputs, "float32")
    engine = engine_factory(world)
    engine.set_option("fuse_staging", fuse)
    engine.set_option("mode", "auto")
    try:
        for r, j in enumerate(jsons):
            engine.register_operation_json("alias", j, r)
        dev = [x.cuda() for x in inputs]
        outs = engine.execute_operation("alias", dev, dev)
    finally:
        engine.set_option("fuse_staging", 1)
    for r in range(world):
        assert bits_equal(outs[r], expect[r]), mismatch_report(outs[r], expect[r])


def test_fused_staging_covers_positions_outside_every_op(engine_factory):
    """A graph that touches only the middle of the tensor: head and tail are passed through."""
    from pccl_amd.dsl import CommunicationOp, compile_to_json_string
    world, n = 2, 4099
    jsons = []
    for rank in range(world):
        other = 1 - rank
        with CommunicationOp(name=f"mid{rank}") as op:
            op.tensor(dtype="float32", shape=(n,))
            op.notify(signal_id=rank, target_rank=other)
            op.wait_notify(signal_id=other, source_rank=other)
            if rank == 0:
                op.sm_reduce(source_rank=1, src_offset=1001, dst_offset=1001, remote_offset=1001, count=2003)
            op.notify(signal_id=10 + rank, target_rank=other)
            op.wait_notify(signal_id=10 + other, source_rank=other)
        g = op.get_graph()
        g.collective_type = "allreduce"
        jsons.append(compile_to_json_string(g))
    inputs = seeded_inputs("randn", world, n, "float32", seed=9)
    expect = oracle_buffers(jsons, inputs, "float32")
    got, info = run_gpu(engine_factory(world), jsons, inputs, "column")
    assert info["num_segments"] == 1
    for r in range(world):
        assert bits_equal(got[r], expect[r]), mismatch_report(got[r], expect[r])
