"""Engine facade on the GPU: the reference's call shapes (pccl/engine.py:11-71,
tests/test_correctness.py:92-104) and the error behaviour of the boundary."""
import json
import os

import pytest
import torch

from helpers import bits_equal, graph_jsons, oracle_buffers, seeded_inputs
from pccl_amd import engine as engine_mod
from pccl_amd._lib import ERR_INVALID, ERR_LINK, ERR_NOT_FOUND, ERR_UNSUPPORTED, PcclError

pytestmark = pytest.mark.gpu


def write_graphs(tmp_path, stem, jsons):
    for r, j in enumerate(jsons):
        (tmp_path / f"{stem}_rank{r}.json").write_text(j)
    return str(tmp_path / (stem + "_rank{rank}.json"))


def test_reference_style_per_rank_flow(engine_factory, tmp_path):
    """register per rank from files, post execute_operation_async per rank, sync, compare."""
    world, n = 4, 1 << 14
    jsons = graph_jsons("ring", "build_allreduce", world, n, "bfloat16", "tma", 1)
    pattern = write_graphs(tmp_path, "ar", jsons)
    eng = engine_factory(world)
    for r in range(world):
        assert eng.rank(r).register_operation("test_allreduce", pattern.format(rank=r)) is True
    inp = [torch.ones(n, dtype=torch.bfloat16, device="cuda") * (r + 1) for r in range(world)]
    out = [torch.zeros_like(t) for t in inp]
    for r in range(world):
        eng.rank(r).execute_operation_async("test_allreduce", inp[r], out[r])
    eng.sync_operation("test_allreduce")
    torch.cuda.synchronize()
    for r in range(world):
        assert (out[r] != world * (world + 1) / 2).sum().item() == 0
    eng.reset_signals("test_allreduce")            # no counts are left here: nothing to clear, must not fail
    # a second round reuses the registration; the last rank may use the synchronising form
    for r in range(world - 1):
        eng.rank(r).execute_operation_async("test_allreduce", inp[r], out[r])
    res = eng.rank(world - 1).execute_operation("test_allreduce", inp[world - 1], out[world - 1])
    assert res is out[world - 1] and (res != 10).sum().item() == 0
    # a synchronising call before the others have posted cannot complete
    with pytest.raises(RuntimeError, match="would block"):
        eng.rank(0).execute_operation("test_allreduce", inp[0], out[0])


def test_collective_form_with_placeholder_and_stacked_tensor(engine_factory, tmp_path):
    world, n = 4, 4096
    jsons = graph_jsons("rhd", "build_allreduce", world, n, "float32", "sm", 1)
    eng = engine_factory(world)
    assert eng.register_operation("rhd", write_graphs(tmp_path, "rhd", jsons)) is True
    x = seeded_inputs("randn", world, n, "float32", seed=21)
    want = oracle_buffers(jsons, x, "float32")
    outs = eng.execute_operation("rhd", torch.stack(x).cuda())     # [R, N] tensor, outputs allocated
    for r in range(world):
        assert bits_equal(outs[r], want[r])
    outs = eng.execute_operation_async("rhd", [t.cuda() for t in x])
    eng.sync_operation("rhd")
    assert bits_equal(outs[2], want[2])
    info = eng.op_info("rhd")
    assert info["num_vranks"] == world and info["num_levels"] == 4


def test_module_level_api(tmp_path):
    world, n = 2, 2048
    jsons = graph_jsons("ring", "build_allreduce", world, n, "float16", "sm", 1)
    pattern = write_graphs(tmp_path, "m", jsons)
    engine_mod.initialize_engine(num_vranks=world)
    try:
        assert engine_mod.register_operation("m", pattern) is True
        x = [torch.full((n,), float(r + 1), dtype=torch.float16, device="cuda") for r in range(world)]
        outs = engine_mod.execute_operation("m", x)
        assert all(torch.all(o == 3) for o in outs)
        engine_mod.sync_operation("m")
        engine_mod.reset_signals("m")
    finally:
        engine_mod.get_engine().close()
        engine_mod._engine_instance = None


def test_registration_and_lookup_errors(engine_factory, tmp_path):
    eng = engine_factory(2)
    assert eng.register_operation("nofile", str(tmp_path / "missing_rank{rank}.json")) is False   # reference: regOp -> false
    (tmp_path / "bad_rank0.json").write_text('{"version": 2}')
    assert eng.register_operation("bad", str(tmp_path / "bad_rank0.json"), rank=0) is False
    doc = json.loads(graph_jsons("ring", "build_allreduce", 2, 2048, "float32", "sm")[0])
    doc["operations"][2]["primitive"] = "sm.scatter"
    (tmp_path / "prim_rank0.json").write_text(json.dumps(doc))
    with pytest.raises(PcclError, match="unknown primitive"):
        eng.register_operation("prim", str(tmp_path / "prim_rank0.json"), rank=0)
    with pytest.raises(PcclError) as e:
        eng.register_operation_json("x", "{}", 7)
    assert e.value.code == ERR_INVALID or "operations" in str(e.value)
    x = [torch.zeros(16, device="cuda") for _ in range(2)]
    with pytest.raises(PcclError, match="Unknown operation") as e:
        eng.execute_operation("never_registered", x)
    assert e.value.code == ERR_NOT_FOUND
    eng.sync_operation("never_registered")                    # the reference returns silently
    with pytest.raises(ValueError, match="expected 2 tensors"):
        eng.execute_operation("never_registered", x[:1])
    with pytest.raises(ValueError, match="GPU"):
        eng.execute_operation("never_registered", [t.cpu() for t in x])
    with pytest.raises(PcclError):
        eng.set_option("mode", "warp-speed")


def test_link_errors_surface_at_first_execution(engine_factory):
    from pccl_amd.dsl import CommunicationOp, compile_to_json_string
    eng = engine_factory(2)
    # only one of two ranks registered
    eng.register_operation_json("half", graph_jsons("ring", "build_allreduce", 2, 2048, "float32", "sm")[0], 0)
    x = [torch.zeros(2048, device="cuda") for _ in range(2)]
    with pytest.raises(PcclError, match="no registered graph") as e:
        eng.execute_operation("half", x)
    assert e.value.code == ERR_LINK
    # a wait nobody releases: reported, not hung
    for rank in range(2):
        with CommunicationOp(name=f"dl{rank}") as op:
            op.tensor(dtype="float32", shape=(2048,))
            op.wait_notify(signal_id=5, source_rank=1 - rank)
            op.sm_copy(source_rank=1 - rank, src_offset=0, dst_offset=0, size=2048)
        eng.register_operation_json("deadlock", compile_to_json_string(op.get_graph()), rank)
    with pytest.raises(PcclError, match="deadlock"):
        eng.execute_operation("deadlock", x)


def test_buffer_checks_and_mode_selection(engine_factory):
    world, n = 2, 4096
    jsons = graph_jsons("ring", "build_allreduce", world, n, "float32", "sm")
    eng = engine_factory(world)
    for r, j in enumerate(jsons):
        eng.register_operation_json("ar", j, r)
    x = seeded_inputs("randn", world, n, "float32", seed=4)
    want = oracle_buffers(jsons, x, "float32")
    small = [torch.zeros(n // 2, device="cuda") for _ in range(world)]
    with pytest.raises(PcclError, match="smaller than"):
        eng.execute_inplace("ar", small, sync=True)
    one_small = [torch.zeros(n, device="cuda"), torch.zeros(n // 2, device="cuda")]   # any rank counts
    with pytest.raises(PcclError, match="smaller than"):
        eng.execute_inplace("ar", one_small, sync=True)
    # buffers that are only 4-byte aligned: auto falls back to the level runner, column refuses
    base = [torch.zeros(n + 4, device="cuda") for _ in range(world)]
    shifted = [b[1:n + 1] for b in base]
    for s, t in zip(shifted, x):
        s.copy_(t)
    eng.set_option("mode", "auto")
    eng.execute_inplace("ar", shifted, sync=True)
    for r in range(world):
        assert bits_equal(shifted[r], want[r])
    eng.set_option("mode", "column")
    with pytest.raises(PcclError, match="16-byte aligned") as e:
        eng.execute_inplace("ar", shifted, sync=True)
    assert e.value.code == ERR_UNSUPPORTED
    eng.set_option("mode", "auto")
    # staged call on the same misaligned tensors (direct plan does not apply, staging does)
    for s, t in zip(shifted, x):
        s.copy_(t)
    outs = eng.execute_operation("ar", shifted)
    for r in range(world):
        assert bits_equal(outs[r], want[r])


def test_column_mode_refuses_graphs_that_are_not_position_aligned(engine_factory):
    world, n = 4, 4096
    eng = engine_factory(world)
    for r, j in enumerate(graph_jsons("ring", "build_alltoall", world, n, "bfloat16")):
        eng.register_operation_json("a2a", j, r)
    eng.set_option("mode", "column")
    x = [torch.zeros(n, dtype=torch.bfloat16, device="cuda") for _ in range(world)]
    with pytest.raises(PcclError, match="same element positions"):
        eng.execute_operation("a2a", x)
    eng.set_option("mode", "auto")
    eng.execute_operation("a2a", x)


def test_kernel_timing_option(engine_factory):
    world, n = 8, 1 << 20
    eng = engine_factory(world)
    for r, j in enumerate(graph_jsons("ring", "build_allreduce", world, n, "bfloat16", "sm", 4)):
        eng.register_operation_json("t", j, r)
    bufs = [torch.zeros(n, dtype=torch.bfloat16, device="cuda") for _ in range(world)]
    with pytest.raises(PcclError, match="timing"):
        eng.last_kernel_ms("t")
    eng.set_option("timing", 1)
    eng.execute_inplace("t", bufs, sync=True)
    ms = eng.last_kernel_ms("t")
    eng.set_option("timing", 0)
    assert 0.0 < ms < 50.0


def test_profiler_ranges_option(engine_factory):
    """The reference wraps the stages of a call in NVTX ranges (engine_c.cc:468-489, cuda_device.cc:313-319);
    here they are roctx ranges behind an option.  Without a profiler attached they must change nothing:
    staged and in-place calls in every mode give the bits they give without them."""
    world, n = 4, 1 << 14
    jsons = graph_jsons("ring", "build_allreduce", world, n, "float32", "sm", 2)
    x = seeded_inputs("randn", world, n, "float32", seed=21)
    want = oracle_buffers(jsons, x, "float32")
    eng = engine_factory(world)
    for r, j in enumerate(jsons):
        eng.register_operation_json("ranges", j, r)
    eng.set_option("trace_ranges", 1)
    try:
        for mode in ("auto", "stepwise", "persistent"):
            eng.set_option("mode", mode)
            for fuse in (1, 0):
                eng.set_option("fuse_staging", fuse)
                outs = eng.execute_operation("ranges", [t.cuda() for t in x])
                bufs = [t.cuda() for t in x]
                eng.execute_inplace("ranges", bufs, sync=True)
                for r in range(world):
                    assert bits_equal(outs[r].cpu(), want[r]) and bits_equal(bufs[r].cpu(), want[r]), (mode, fuse, r)
    finally:
        eng.set_option("trace_ranges", 0)
        eng.set_option("fuse_staging", 1)
        eng.set_option("mode", "auto")


def test_info_log_lines_of_registration_and_linking():
    """The reference logs engine start, registration and the runner it picked at INFO
    (engine_c.cc:84,163,168,199,357); the same three moments are logged here, on stderr."""
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    code = (
        "import sys; sys.path[:0] = [%r, %r]\n"
        "import torch\n"
        "from helpers import graph_jsons\n"
        "from pccl_amd.engine import Engine\n"
        "e = Engine(2, 0)\n"
        "for r, j in enumerate(graph_jsons('ring', 'build_allreduce', 2, 4096, 'float32', 'sm', 1)):\n"
        "    e.register_operation_json('logged', j, r)\n"
        "b = [torch.ones(4096, device='cuda') for _ in range(2)]\n"
        "e.execute_inplace('logged', b, sync=True)\n"
        "print('sum', float(b[0][0]))\n"
        "e.close()\n") % (root, os.path.join(root, "tests"))
    env = dict(os.environ, PCCL_LOG_LEVEL="INFO")
    out = subprocess.run([sys.executable, "-c", code], env=env, capture_output=True, text=True, timeout=300)
    assert out.returncode == 0, out.stderr
    assert out.stdout.strip().splitlines()[-1] == "sum 2.0"
    assert "[pccl] [info] engine context on device 0 with 2 virtual ranks" in out.stderr
    assert "[pccl] [info] operation 'logged' registered for virtual rank 1: " in out.stderr
    assert "[pccl] [info] linked 2 rank graphs: 4 data ops on 2 levels" in out.stderr and "slot runner with 256 threads" in out.stderr


def test_registration_from_trigger_arrays(engine_factory):
    """What a C++ engine that parses the JSON itself would hand over: the 32-byte triggers and the
    88-byte metadata records (reference proxy_trigger.h:8-16, primitive.h:8-17)."""
    from pccl_amd import _lib
    from pccl_amd._lib import HostGraph
    world, n = 4, 1 << 13
    jsons = graph_jsons("ring", "build_allreduce", world, n, "bfloat16", "sm", 2)
    eng = engine_factory(world)
    for r, j in enumerate(jsons):
        g = HostGraph.from_json(j)
        trig, cnt = g.triggers()
        meta, _ = g.meta()
        _lib.check(eng._L.pccl_hip_register_triggers(eng._h, b"trig", r, trig, meta, cnt, b"allreduce"))
    x = seeded_inputs("randn", world, n, "bfloat16", seed=8)
    want = oracle_buffers(jsons, x, "bfloat16")
    outs = eng.execute_operation("trig", [t.cuda() for t in x])
    for r in range(world):
        assert bits_equal(outs[r], want[r])


def test_reregistration_replaces_the_operation_and_operations_share_the_rank_buffers(engine_factory):
    """Registering a name again replaces its graphs (the next execution links the new ones); every
    operation of an engine aliases the same rank buffers (reference engine_c.cc:191-196), which grow
    with the largest graph registered and keep working for the smaller ones."""
    world = 4
    eng = engine_factory(world)
    eng.set_option("fuse_staging", 0)           # go through the engine's rank buffers
    try:
        cases = {}
        for name, alg, n, dtype in (("a", "ring", 1 << 12, "float32"), ("b", "rhd", 1 << 16, "float32")):
            jsons = graph_jsons(alg, "build_allreduce", world, n, dtype, "sm", 1)
            for r, j in enumerate(jsons):
                eng.register_operation_json(name, j, r)
            x = seeded_inputs("randn", world, n, dtype, seed=len(cases) + 1)
            cases[name] = (jsons, x, oracle_buffers(jsons, x, dtype))
        for name in ("a", "b", "a", "b"):
            jsons, x, want = cases[name]
            outs = eng.execute_operation(name, [t.cuda() for t in x])
            assert all(bits_equal(o, w) for o, w in zip(outs, want)), name
        # replace "a" by a tree on a different size
        n2 = 3000
        jsons = graph_jsons("tree", "build_allreduce", world, n2, "float32", "sm", 1)
        for r, j in enumerate(jsons):
            eng.register_operation_json("a", j, r)
        x = seeded_inputs("uniform", world, n2, "float32", seed=9)
        want = oracle_buffers(jsons, x, "float32")
        outs = eng.execute_operation("a", [t.cuda() for t in x])
        assert all(bits_equal(o, w) for o, w in zip(outs, want))
        assert eng.op_info("a")["num_data_ops"] == 2 * (world - 1)
        jsons_b, xb, want_b = cases["b"]
        outs = eng.execute_operation("b", [t.cuda() for t in xb])
        assert all(bits_equal(o, w) for o, w in zip(outs, want_b))
    finally:
        eng.set_option("fuse_staging", 1)


def test_executions_follow_the_callers_stream(engine_factory):
    """Kernels are enqueued on the current torch stream (reference cuda_device.cc:245-248,301): work
    queued on a side stream before and after the call is ordered with it."""
    world, n = 2, 1 << 20
    jsons = graph_jsons("ring", "build_allreduce", world, n, "float32", "sm", 1)
    eng = engine_factory(world)
    for r, j in enumerate(jsons):
        eng.register_operation_json("s", j, r)
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        x = [torch.full((n,), float(r + 1), device="cuda") for r in range(world)]   # produced on the side stream
        outs = eng.execute_operation_async("s", x)
        y = outs[0] * 2                                                             # consumed on it
    side.synchronize()
    assert torch.all(y == 6) and torch.all(outs[1] == 3)


def test_prepared_calls(engine_factory):
    """Engine.prepare binds an operation to fixed tensors; every invocation is just the C call."""
    world, n = 8, 4096
    chunk = n // world
    jsons = graph_jsons("ring", "build_reduce_scatter", world, n, "float16", "sm", 1)
    eng = engine_factory(world)
    for r, j in enumerate(jsons):
        eng.register_operation_json("rs", j, r)
    x = seeded_inputs("randn0.1", world, n, "float16", seed=6)
    want = oracle_buffers(jsons, x, "float16")
    ins = [t.cuda() for t in x]
    outs = [torch.zeros(chunk, dtype=torch.float16, device="cuda") for _ in range(world)]
    call = eng.prepare("rs", ins, outs)
    for _ in range(3):
        for o in outs:
            o.zero_()
        got = call(sync=True)
        for r in range(world):
            assert got[r] is outs[r] and bits_equal(outs[r], want[r][r * chunk:(r + 1) * chunk])
    # in place, on an explicit stream handle
    ar = graph_jsons("ring", "build_allreduce", world, n, "float16", "sm", 1)
    for r, j in enumerate(ar):
        eng.register_operation_json("ar", j, r)
    bufs = [t.cuda() for t in x]
    call = eng.prepare("ar", bufs)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    call(stream=side.cuda_stream)
    side.synchronize()
    want = oracle_buffers(ar, x, "float16")
    for r in range(world):
        assert bits_equal(bufs[r], want[r])
    with pytest.raises(ValueError, match="expected 8 tensors"):
        eng.prepare("ar", bufs[:3])


@pytest.mark.parametrize("mode", ["auto", "stepwise", "persistent"])
def test_executions_can_be_captured_into_a_graph_of_the_caller(engine_factory, mode):
    """After a first eager execution (linking and table upload allocate) an execution is kernel
    launches only, so a caller may capture it into a graph (the persistent runner then takes its
    launch number from a device-side counter, since a replay repeats the kernel arguments).  Every
    replay is checked against the oracle, with eager work and synchronisations in between, and so is
    an eager execution after the replays."""
    world, n = 8, 1 << 16
    jsons = graph_jsons("ring", "build_allreduce", world, n, "bfloat16", "sm", 2)
    eng = engine_factory(world)
    for r, j in enumerate(jsons):
        eng.register_operation_json("ar", j, r)
    eng.set_option("mode", mode)
    x = seeded_inputs("randn", world, n, "bfloat16", seed=11)
    want = oracle_buffers(jsons, x, "bfloat16")
    src = [t.cuda() for t in x]
    bufs = [torch.empty_like(t) for t in src]
    for b, t in zip(bufs, src):
        b.copy_(t)
    eng.execute_inplace("ar", bufs, sync=True)          # eager: links, uploads, and is the reference run
    for r in range(world):
        assert bits_equal(bufs[r], want[r])
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            for b, t in zip(bufs, src):
                b.copy_(t)
            eng.execute_inplace("ar", bufs)
    torch.cuda.current_stream().wait_stream(side)
    for rep in range(4):
        for b in bufs:
            b.fill_(float(rep))                           # eager work between the replays
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        for r in range(world):
            assert bits_equal(bufs[r], want[r]), f"replay {rep}, rank {r}"
    for b, t in zip(bufs, src):
        b.copy_(t)
    eng.execute_inplace("ar", bufs, sync=True)
    for r in range(world):
        assert bits_equal(bufs[r], want[r]), f"eager execution after the replays, rank {r}"


def test_calls_from_several_threads(engine_factory):
    """One context, four host threads, each with its own stream and tensors, two operations: the
    context's mutex serialises registration, linking and launches; results stay exact."""
    import threading
    world, n = 4, 1 << 14
    eng = engine_factory(world)
    specs = {"ar_f32": ("float32", 1), "ar_bf16": ("bfloat16", 2)}
    want, inputs = {}, {}
    for name, (dtype, ch) in specs.items():
        jsons = graph_jsons("ring", "build_allreduce", world, n, dtype, "sm", ch)
        for r, j in enumerate(jsons):
            eng.register_operation_json(name, j, r)
        inputs[name] = seeded_inputs("randn", world, n, dtype, seed=21)
        want[name] = oracle_buffers(jsons, inputs[name], dtype)
    errors = []

    def worker(k):
        try:
            name = list(specs)[k % 2]
            stream = torch.cuda.Stream()
            src = [t.cuda() for t in inputs[name]]
            with torch.cuda.stream(stream):
                for it in range(25):
                    bufs = [t.clone() for t in src]
                    if it % 2:
                        eng.execute_inplace(name, bufs)
                        got = bufs
                    else:
                        got = eng.execute_operation_async(name, bufs)
                    stream.synchronize()
                    for r in range(world):
                        if not bits_equal(got[r], want[name][r]):
                            raise AssertionError(f"thread {k}, iteration {it}, rank {r}")
        except Exception as e:   # noqa: BLE001 - reported by the main thread
            errors.append(repr(e))

    threads = [threading.Thread(target=worker, args=(k,)) for k in range(4)]
    for t in threads:
        t.start()
    for t in threads:
        t.join(timeout=100)
    assert not any(t.is_alive() for t in threads), "a worker thread did not finish"
    assert not errors, errors


def test_tensors_of_the_wrong_element_size_are_refused(engine_factory):
    world, n = 2, 2048
    eng = engine_factory(world)
    for r, j in enumerate(graph_jsons("ring", "build_allreduce", world, n, "bfloat16", "sm")):
        eng.register_operation_json("ar_bf16_only", j, r)
    wrong = [torch.zeros(n, device="cuda", dtype=torch.float32) for _ in range(world)]
    with pytest.raises(ValueError, match="4-byte elements"):
        eng.execute_inplace("ar_bf16_only", wrong)
    with pytest.raises(ValueError, match="4-byte elements"):
        eng.execute_operation("ar_bf16_only", wrong)
    right = [torch.ones(n, device="cuda", dtype=torch.bfloat16) for _ in range(world)]
    eng.execute_inplace("ar_bf16_only", right, sync=True)
    assert torch.all(right[0].float() == 2)
    as_int16 = [t.view(torch.int16) for t in right]          # same element size: the bytes are what counts
    eng.execute_inplace("ar_bf16_only", as_int16, sync=True)
    assert torch.all(right[1].float() == 4)


OPTIONS = {   # key: (values that are taken and read back as written, values that are refused)
    "mode": (["column", "stepwise", "persistent", "auto"], ["fast", ""]),
    "num_blocks": ([7, 0], ["many"]),
    "timing": ([1, 0], ["on"]),
    "fuse_staging": ([0, 1], ["yes"]),
    "wait_timeout_ms": ([5, 2000], ["1s"]),
    "check_races": ([0, 1], ["no"]),
    "vecs_per_thread": ([2, 4, 1], [3, 0, "two"]),
    "slot_direct": ([0, 1], ["direct"]),
    "slot_store_waves": ([0, 1, -1], [2, -2]),
    "level_graph": ([1, 0], ["graph"]),
    "phased": ([0, 1, -1], [2, -2, "always"]),
    "phased_shape": ([0, 1, -1], [2, 4]),
    "phased_exchange": ([0, 1, -1], [2]),
    "phased_sweeps": ([1, 2, -1], [0, 3, "two"]),
    "phased_linear": ([0, 1, -1], [2, -2]),
    "phased_barriers": ([0, 1], ["x"]),
    "phased_timeout_us": ([50, 1000], ["1ms"]),
    "lds_slots": ([0, 1], ["lds"]),
    "slot_threads": ([64, 512, 0], [100, 2048]),
    "slot_vecs": ([2, 1, 0], [3, 8]),
    "slot_lds_kib": ([96, 0], [161, -1, "64k"]),
    "step_tile_bytes": ([8192, 0], [1000, -4096, "4k"]),
}


def test_every_option_reads_back_and_refuses_what_it_cannot_take(engine_factory):
    """set_option / get_option over every key of the header: a value that is taken reads back as it
    was written, a value that is refused (out of range, not a whole number) raises with the key's name
    or its range in the message and leaves the option as it was, True and False arrive as 1 and 0, and
    an unknown key is an error for both calls."""
    eng = engine_factory(4)
    for key, (good, bad) in OPTIONS.items():
        start = eng.get_option(key)
        try:
            for v in good:
                eng.set_option(key, v)
                assert eng.get_option(key) == str(v), key
            kept = eng.get_option(key)
            for v in bad:
                with pytest.raises(PcclError) as e:
                    eng.set_option(key, v)
                assert e.value.code == ERR_INVALID, (key, v)
                assert key in str(e.value) or "must be" in str(e.value), str(e.value)
                assert eng.get_option(key) == kept, (key, v)
        finally:
            eng.set_option(key, start)
    eng.set_option("timing", True)
    assert eng.get_option("timing") == "1"
    eng.set_option("timing", False)
    assert eng.get_option("timing") == "0"
    for call in (lambda: eng.set_option("no_such_option", 1), lambda: eng.get_option("no_such_option")):
        with pytest.raises(PcclError, match="unknown option") as e:
            call()
        assert e.value.code == ERR_INVALID
    assert eng.get_option("num_vranks") == "4"
    with pytest.raises(PcclError, match="Unknown operation"):
        eng.get_option("slot_shape:nobody")
