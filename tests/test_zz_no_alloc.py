"""pccl_hip_execute_inplace_static: the in-place execution for callers that cannot allocate.  Called
through the C ABI and compared bit for bit with the CPU oracle and with pccl_hip_execute_inplace on
the same inputs, on calls in a row that share the GPU's static workspace: a larger operation, then a smaller one (whose
tables replace the first one's and whose flags must not be confused with what the first left
behind), then the first again, then repeated launches of one operation."""
import ctypes

import pytest
import torch

from helpers import bits_equal, graph_jsons, mismatch_report, oracle_buffers, seeded_inputs
from pccl_amd import _lib
from pccl_amd._lib import ERR_INVALID

pytestmark = pytest.mark.gpu


def _ptrs(ts):
    return (ctypes.c_void_p * len(ts))(*[t.data_ptr() for t in ts])


def _stream():
    return torch.cuda.current_stream().cuda_stream


def _register(L, h, name, jsons):
    for r, j in enumerate(jsons):
        data = j.encode()
        _lib.check(L.pccl_hip_register_json(h, name.encode(), r, data, len(data)))


def test_static_workspace_execution_matches_the_allocating_entry_point():
    L = _lib.lib()
    world = 8
    h = ctypes.c_void_p()
    _lib.check(L.pccl_hip_create(ctypes.byref(h), 0, world))
    try:
        cases = {   # name -> (graphs, elements per rank, dtype, input kind)
            "large": (graph_jsons("ring", "build_allreduce", world, 1 << 20, "bfloat16", "sm", 2), 1 << 20, "bfloat16", "randn"),
            "small": (graph_jsons("rhd", "build_allreduce", world, 3 * 4096, "float32", "sm", 1), 3 * 4096, "float32", "randn"),
            "tree": (graph_jsons("tree", "build_allreduce", world, 40000, "int32", "sm", 1, reduce_op="max"), 40000, "int32", "randint"),
        }
        inputs, want, oracle_want = {}, {}, {}
        for name, (jsons, n, dtype, kind) in cases.items():
            _register(L, h, name, jsons)
            host = seeded_inputs(kind, world, n, dtype, seed=len(name))
            oracle_want[name] = oracle_buffers(jsons, host, dtype)
            inputs[name] = [t.cuda() for t in host]

        def run_static(name, bufs=None):
            bufs = bufs if bufs is not None else [t.clone() for t in inputs[name]]
            _lib.check(L.pccl_hip_execute_inplace_static(h, name.encode(), _ptrs(bufs), bufs[0].nbytes, _stream(), 1))
            return bufs

        # the static entry point first, on operations that have never been linked on the device
        print("static: large, then small, then large again", flush=True)
        got = {"large": run_static("large")}
        got["small"] = run_static("small")            # the second call, on a smaller input
        got["large2"] = run_static("large")
        got["tree"] = run_static("tree")
        torch.cuda.synchronize()
        for key, bufs in got.items():
            name = "large" if key == "large2" else key
            for r in range(world):
                assert bits_equal(bufs[r], oracle_want[name][r]), f"{key} vs the oracle, rank {r}: {mismatch_report(bufs[r], oracle_want[name][r])}"

        # Nothing is allocated: with every kernel of the path loaded by the calls above, alternating
        # calls - each takes the workspace over from the other: fill, table-write and map kernels -
        # on buffers made beforehand leave the device's free memory exactly where it was.
        held = {name: [t.clone() for t in inputs[name]] for name in cases}
        torch.cuda.synchronize()
        free_before = torch.cuda.mem_get_info()[0]
        for i in range(6):
            for name in ("large", "small", "tree"):
                run_static(name, held[name])
        torch.cuda.synchronize()
        assert torch.cuda.mem_get_info()[0] == free_before, "the static entry point allocated device memory"
        del held

        # the existing entry point on the same inputs (persistent runner and the default runner)
        for mode in ("persistent", "auto"):
            _lib.check(L.pccl_hip_set_option(h, b"mode", mode.encode()))
            for name in cases:
                bufs = [t.clone() for t in inputs[name]]
                _lib.check(L.pccl_hip_execute_inplace(h, name.encode(), _ptrs(bufs), bufs[0].nbytes, _stream(), 1))
                want[name] = bufs
                keys = [name, "large2"] if name == "large" else [name]
                for key in keys:
                    for r in range(world):
                        assert bits_equal(got[key][r], bufs[r]), f"{key} vs execute_inplace ({mode}), rank {r}: {mismatch_report(got[key][r], bufs[r])}"

        # many launches in a row of one operation, alternating with another: flags of earlier launches
        # must never satisfy a later one
        print("static: 40 launches alternating between two operations", flush=True)
        for i in range(40):
            name = "small" if i % 3 else "tree"
            bufs = run_static(name)
            for r in range(world):
                assert bits_equal(bufs[r], want[name][r]), f"launch {i} ({name}), rank {r}"

        # asynchronous launches followed by pccl_hip_sync
        bufs = [t.clone() for t in inputs["small"]]
        _lib.check(L.pccl_hip_execute_inplace_static(h, b"small", _ptrs(bufs), bufs[0].nbytes, _stream(), 0))
        _lib.check(L.pccl_hip_sync(h, b"small"))
        for r in range(world):
            assert bits_equal(bufs[r], want["small"][r])

        # limits: rank buffers too small, and an operation whose tables exceed the workspace
        small_bufs = [t[:100].clone() for t in inputs["large"]]
        assert L.pccl_hip_execute_inplace_static(h, b"large", _ptrs(small_bufs), small_bufs[0].nbytes, _stream(), 1) == ERR_INVALID
        assert b"smaller than" in L.pccl_hip_last_error()
        _lib.check(L.pccl_hip_set_option(h, b"step_tile_bytes", b"4096"))
        _register(L, h, "huge", graph_jsons("ring", "build_allreduce", world, 1 << 27, "bfloat16", "sm", 4))
        rc = L.pccl_hip_execute_inplace_static(h, b"huge", _ptrs(small_bufs), small_bufs[0].nbytes, _stream(), 1)
        assert rc == ERR_INVALID and b"static workspace holds" in L.pccl_hip_last_error(), L.pccl_hip_last_error()
        assert L.pccl_hip_execute_inplace_static(h, b"nope", _ptrs(small_bufs), 200, _stream(), 1) == _lib.ERR_NOT_FOUND
    finally:
        L.pccl_hip_destroy(h)


def test_recorded_launches_and_a_workspace_that_changes_hands():
    """The entry point under graph capture, the case it exists for.  After one eager call the
    operation's tables sit in the workspace and a call is kernel launches only: it is recorded into
    a graph of the caller and every replay is compared with pccl_hip_execute_inplace, with eager
    work and synchronisations between the replays.  Then another operation takes the workspace over.
    A replay of the old graph now finds foreign tables behind its kernel arguments: it must execute
    nothing (the buffers keep what they held); the call that notices it - another operation's - is
    not failed, and the first operation's next pccl_hip_sync reports it.  After an eager call of the
    first operation the same graph works again."""
    L = _lib.lib()
    world, n = 8, 1 << 16
    h = ctypes.c_void_p()
    _lib.check(L.pccl_hip_create(ctypes.byref(h), 0, world))
    try:
        jsons_a = graph_jsons("ring", "build_allreduce", world, n, "bfloat16", "sm", 2)
        _register(L, h, "a", jsons_a)
        _register(L, h, "b", graph_jsons("rhd", "build_allreduce", world, 4096, "float32", "sm", 1))
        host_src = seeded_inputs("randn", world, n, "bfloat16", seed=21)
        src = [t.cuda() for t in host_src]
        want = [t.clone() for t in src]
        _lib.check(L.pccl_hip_execute_inplace(h, b"a", _ptrs(want), want[0].nbytes, _stream(), 1))
        for r, o in enumerate(oracle_buffers(jsons_a, host_src, "bfloat16")):
            assert bits_equal(want[r], o), f"execute_inplace vs the oracle, rank {r}: {mismatch_report(want[r], o)}"
        bufs = [t.clone() for t in src]
        _lib.check(L.pccl_hip_execute_inplace_static(h, b"a", _ptrs(bufs), bufs[0].nbytes, _stream(), 1))
        for r in range(world):
            assert bits_equal(bufs[r], want[r]), mismatch_report(bufs[r], want[r])

        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.stream(side):
            with torch.cuda.graph(graph, stream=side):
                for b, t in zip(bufs, src):
                    b.copy_(t)
                _lib.check(L.pccl_hip_execute_inplace_static(h, b"a", _ptrs(bufs), bufs[0].nbytes, side.cuda_stream, 0))
        torch.cuda.current_stream().wait_stream(side)
        for rep in range(3):
            print(f"replay {rep}", flush=True)
            for b in bufs:
                b.fill_(float(rep))                       # eager work between the replays
            torch.cuda.synchronize()
            graph.replay()
            torch.cuda.synchronize()
            for r in range(world):
                assert bits_equal(bufs[r], want[r]), f"replay {rep}, rank {r}"

        print("another operation takes the workspace, then the old graph is replayed", flush=True)
        other = [t.cuda() for t in seeded_inputs("randn", world, 4096, "float32", seed=22)]
        _lib.check(L.pccl_hip_execute_inplace_static(h, b"b", _ptrs(other), other[0].nbytes, _stream(), 1))
        graph.replay()                                    # copies the inputs in, then a launch that must do nothing
        torch.cuda.synchronize()
        for r in range(world):
            assert bits_equal(bufs[r], src[r]), f"a stale replay touched rank {r}"
        # the operation that owns the workspace now runs normally and gives the same result as before
        first_b = [t.clone() for t in other]
        other2 = [t.cuda() for t in seeded_inputs("randn", world, 4096, "float32", seed=22)]
        _lib.check(L.pccl_hip_execute_inplace_static(h, b"b", _ptrs(other2), other2[0].nbytes, _stream(), 1))
        for r in range(world):
            assert bits_equal(other2[r], first_b[r]), "the call that noticed the stale replay did not execute normally"
        _lib.check(L.pccl_hip_sync(h, b"b"))
        # the operation whose recorded launch it was hears of it at its own sync, once
        assert L.pccl_hip_sync(h, b"a") == ERR_INVALID
        msg = L.pccl_hip_last_error()
        assert b"operation 'a'" in msg and b"executed nothing" in msg and b"unchanged" in msg, msg
        _lib.check(L.pccl_hip_sync(h, b"a"))

        print("the first operation again, eagerly and from the graph", flush=True)
        again = [t.clone() for t in src]
        _lib.check(L.pccl_hip_execute_inplace_static(h, b"a", _ptrs(again), again[0].nbytes, _stream(), 1))
        for r in range(world):
            assert bits_equal(again[r], want[r])
        graph.replay()
        torch.cuda.synchronize()
        for r in range(world):
            assert bits_equal(bufs[r], want[r]), f"replay after the workspace came back, rank {r}"
        _lib.check(L.pccl_hip_sync(h, b"a"))
    finally:
        _lib.check(L.pccl_hip_destroy(h))
