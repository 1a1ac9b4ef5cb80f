"""Corners of the boundary on the GPU: the environment switches the reference reads, set-up work
refused on a capturing stream, the column runners' hand-written store under the pattern it has to
survive, and the shapes of workgroup the slot runner can be given."""
import json
import os
import subprocess
import sys

import pytest
import torch

from helpers import (ROOT, bits_equal, graph_jsons, mismatch_report, oracle_buffers, random_program, seeded_inputs)
from pccl_amd._lib import ERR_INVALID, PcclError
from pccl_amd.dsl import CommunicationOp, compile_to_json_string

pytestmark = pytest.mark.gpu


def test_environment_switches_of_the_reference():
    """PCCL_NUM_BLOCKS and PCCL_DISABLE_FUSED are read where the reference reads them (workgroup count of
    a launch, csrc/plugins/cuda/cuda_device.cc:289-298; fused runner off, csrc/engine_c.cc:351) and
    PCCL_VRANKS gives the number of virtual ranks when the caller does not.  A new context shows what
    they left behind, and the results stay exact: with the fused (column) runner off the level runner
    executes the graph, with 7 workgroups per launch every kernel strides over its tiles."""
    code = ("import sys, json; sys.path.insert(0, %r); sys.path.insert(0, %r)\n"
            "import torch\n"
            "from helpers import graph_jsons, seeded_inputs, oracle_buffers, bits_equal\n"
            "from pccl_amd.engine import Engine\n"
            "eng = Engine()\n"
            "world, n = eng.num_vranks, 40320\n"
            "jsons = graph_jsons('ring', 'build_allreduce', world, n, 'float32', 'sm', 2)\n"
            "for r, j in enumerate(jsons): eng.register_operation_json('ar', j, r)\n"
            "x = seeded_inputs('randn', world, n, 'float32', seed=3)\n"
            "want = oracle_buffers(jsons, x, 'float32')\n"
            "outs = eng.execute_operation('ar', [t.cuda() for t in x])\n"
            "ok = all(bits_equal(outs[r], want[r]) for r in range(world))\n"
            "bufs = [t.cuda() for t in x]\n"
            "eng.execute_inplace('ar', bufs, sync=True)\n"
            "ok = ok and all(bits_equal(bufs[r], want[r]) for r in range(world))\n"
            "print(json.dumps({'vranks': world, 'mode': eng.get_option('mode'), 'num_blocks': eng.get_option('num_blocks'), 'exact': ok}))\n"
            ) % (ROOT, os.path.join(ROOT, "tests"))
    base = {k: v for k, v in os.environ.items() if k not in ("PCCL_NUM_BLOCKS", "PCCL_DISABLE_FUSED", "PCCL_VRANKS")}

    def run(**env):
        print(f"environment {env}", flush=True)
        out = subprocess.run([sys.executable, "-c", code], env={**base, **env}, capture_output=True, text=True, timeout=300)
        assert out.returncode == 0, out.stderr
        return json.loads(out.stdout.strip().splitlines()[-1])

    assert run(PCCL_VRANKS="4") == {"vranks": 4, "mode": "auto", "num_blocks": "0", "exact": True}
    assert run(PCCL_VRANKS="6", PCCL_DISABLE_FUSED="1") == {"vranks": 6, "mode": "stepwise", "num_blocks": "0", "exact": True}
    assert run(PCCL_VRANKS="8", PCCL_NUM_BLOCKS="7") == {"vranks": 8, "mode": "auto", "num_blocks": "7", "exact": True}
    out = subprocess.run([sys.executable, "-c", code], env=base, capture_output=True, text=True, timeout=300)
    assert out.returncode != 0 and "PCCL_VRANKS" in out.stderr       # neither an argument nor the variable


def test_setup_work_is_refused_on_a_capturing_stream(engine_factory):
    """Linking an operation allocates and uploads its plan tables, and a staged call may have to grow
    the engine's rank buffers: on a stream that is being captured either would invalidate the caller's
    capture, so the call is refused with PCCL_ERR_INVALID and nothing is enqueued.  The capture goes
    on; after one eager execution the same call is captured and replays correctly."""
    world, n = 4, 1 << 14
    jsons = graph_jsons("ring", "build_allreduce", world, n, "float32", "sm", 1)
    eng = engine_factory(world)
    for r, j in enumerate(jsons):
        eng.register_operation_json("cap", j, r)
    x = seeded_inputs("randn", world, n, "float32", seed=21)
    want = oracle_buffers(jsons, x, "float32")
    src = [t.cuda() for t in x]
    bufs = [t.clone() for t in src]
    outs = [torch.empty_like(t) for t in src]
    marker = torch.zeros(8, device="cuda")
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            marker.add_(1.0)
            with pytest.raises(PcclError, match="capturing") as e:
                eng.execute_inplace("cap", bufs)           # never linked: would allocate
            assert e.value.code == ERR_INVALID
            assert eng.op_info("cap")["num_data_ops"] == 4 * 6     # inspection links on the host only: allowed
            marker.add_(1.0)
    torch.cuda.current_stream().wait_stream(side)
    graph.replay()
    torch.cuda.synchronize()
    assert marker[0].item() == 2.0                         # the capture survived the refused call
    for r in range(world):
        assert bits_equal(bufs[r], src[r])                 # and nothing ran

    eng.execute_inplace("cap", bufs, sync=True)            # eager: links
    for r in range(world):
        assert bits_equal(bufs[r], want[r])
    # a staged call through the engine's rank buffers, which do not exist yet: refused while capturing
    eng.set_option("mode", "stepwise")
    graph2 = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph2, stream=side):
            marker.add_(1.0)
            with pytest.raises(PcclError, match="capturing"):
                eng.execute_operation_async("cap", src, outs)
    torch.cuda.current_stream().wait_stream(side)
    eng.execute_operation("cap", src, outs)                # eager: allocates the rank buffers
    for r in range(world):
        assert bits_equal(outs[r], want[r])
    graph3 = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph3, stream=side):
            eng.execute_operation_async("cap", src, outs)  # kernels only now
    torch.cuda.current_stream().wait_stream(side)
    for rep in range(3):
        for o in outs:
            o.zero_()
        torch.cuda.synchronize()
        graph3.replay()
        torch.cuda.synchronize()
        for r in range(world):
            assert bits_equal(outs[r], want[r]), f"replay {rep}, rank {r}"
    eng.set_option("mode", "auto")


DTYPES6 = ["float32", "float16", "bfloat16", "int32", "float8_e4m3", "float8_e5m2"]


def _pairs_program(rank, world, n, dtype):
    """Rank 2k+1 reduces from rank 2k and then copies rank 2k's input over a second range; rank 2k does
    nothing.  Position by position the column program is a run of instructions that each load two
    fresh operands, store their result for good and are followed at once by the next instruction,
    which overwrites the registers the store has just read from."""
    half = n // 2
    with CommunicationOp(name=f"pairs_rank{rank}") as op:
        op.tensor(dtype=dtype, shape=(n,))
        if rank % 2 == 1:
            op.sm_reduce(reduce_op="sum", source_rank=rank - 1, remote_offset=0, src_offset=0, dst_offset=0, count=half + 3)
            op.sm_copy(source_rank=rank - 1, src_offset=half + 3, dst_offset=half + 3, size=n - half - 3)
        else:
            op.sm_copy(source_rank=rank, src_offset=0, dst_offset=0, size=0)
        return compile_to_json_string(op.get_graph())


@pytest.mark.parametrize("dtype", DTYPES6)
def test_store_followed_at_once_by_an_overwrite_of_its_data(engine_factory, dtype):
    """The column runners store with a hand-written instruction (a pointer store marked agent scope
    and non-temporal, with the wait state a 128-bit store needs before its data registers may be
    overwritten).  This is the pattern that would break first if that wait state were lost: every
    instruction stores its result and the next one overwrites the same registers immediately; slot
    runner (1, 2 and 4 vectors per thread) and register runner, all six element types, a size that
    leaves cut vectors at the range boundaries."""
    world, n = 16, 3 * 8192 + 5
    jsons = [_pairs_program(r, world, n, dtype) for r in range(world)]
    kind = "randint" if dtype == "int32" else "randn"
    x = seeded_inputs(kind, world, n, dtype, seed=5)
    want = oracle_buffers(jsons, x, dtype)
    eng = engine_factory(world)
    for r, j in enumerate(jsons):
        eng.register_operation_json("pairs", j, r)
    eng.set_option("mode", "column")
    shapes = [("slot", 64, 1), ("slot", 128, 2), ("slot", 64, 4), ("slot", 256, 1), ("register", 0, 1), ("register", 0, 4)]
    try:
        for runner, threads, vecs in shapes:
            print(f"{dtype}: {runner} runner, threads={threads} vecs={vecs}", flush=True)
            if runner == "slot":
                eng.set_option("lds_slots", 1); eng.set_option("slot_vecs", vecs); eng.set_option("slot_threads", threads)
            else:
                eng.set_option("lds_slots", 0); eng.set_option("vecs_per_thread", vecs)
            bufs = [t.cuda() for t in x]
            eng.execute_inplace("pairs", bufs, sync=True)
            for r in range(world):
                assert bits_equal(bufs[r], want[r]), f"{runner} {threads}x{vecs}, rank {r}: {mismatch_report(bufs[r], want[r])}"
    finally:
        for key, val in (("lds_slots", 1), ("slot_threads", 0), ("slot_vecs", 0), ("vecs_per_thread", 1), ("mode", "auto")):
            eng.set_option(key, val)


SLOT_SHAPES = [(64, 1, 0), (64, 4, 0), (128, 2, 0), (256, 4, 0), (512, 1, 96), (512, 2, 0), (1024, 1, 0), (256, 1, 160)]


@pytest.mark.parametrize("seed", [2, 5, 9])
def test_slot_runner_workgroup_shapes(engine_factory, seed):
    """The slot runner's workgroup can be 64 to 1024 threads with 1, 2 or 4 vectors per thread and a
    floor on the LDS it asks for: random race-free aligned programs (odd sizes, so tiles cut by range
    boundaries and cut vectors occur in every shape) must give the oracle's bits in each, in place
    and as a staged ring call on the caller's tensors."""
    world = 3 + seed % 5
    dtype = DTYPES6[seed % 6]
    n = 20000 + 1031 * seed
    red = ("sum",) if dtype.startswith("float8") else ("sum", "max", "min")
    jsons = random_program(2000 + seed, world, n, 60, dtype, True, reduce_ops=red)
    kind = "randint" if dtype == "int32" else "randn"
    x = seeded_inputs(kind, world, n, dtype, seed=seed)
    want = oracle_buffers(jsons, x, dtype)
    ring_n = 8 * world * 250 + 0
    ring = graph_jsons("ring", "build_allreduce", world, ring_n, dtype, "sm", 2)
    rx = seeded_inputs(kind, world, ring_n, dtype, seed=seed + 1)
    ring_want = oracle_buffers(ring, rx, dtype)
    eng = engine_factory(world)
    for r in range(world):
        eng.register_operation_json("rnd", jsons[r], r)
        eng.register_operation_json("ring", ring[r], r)
    eng.set_option("mode", "column")
    try:
        for threads, vecs, kib in SLOT_SHAPES:
            if threads * vecs > 1024 or world * threads * vecs * 16 > 160 * 1024:
                continue
            eng.set_option("slot_vecs", vecs); eng.set_option("slot_threads", threads); eng.set_option("slot_lds_kib", kib)
            # store_waves: the broadcast tail through LDS, whole tiles of a rank stored by one wave;
            # blocks: a grid smaller than the number of tiles, so that workgroups walk several tiles
            for store_waves, blocks in ((0, 0), (1, 0), (1, 5)):
                print(f"seed {seed} {dtype} R={world}: threads={threads} vecs={vecs} lds_kib={kib} store_waves={store_waves} blocks={blocks}", flush=True)
                eng.set_option("slot_store_waves", store_waves); eng.set_option("num_blocks", blocks)
                what = f"{threads}x{vecs} store_waves={store_waves} blocks={blocks}"
                bufs = [t.cuda() for t in x]
                eng.execute_inplace("rnd", bufs, sync=True)
                for r in range(world):
                    assert bits_equal(bufs[r], want[r]), f"{what}, rank {r}: {mismatch_report(bufs[r], want[r])}"
                outs = eng.execute_operation("ring", [t.cuda() for t in rx])
                for r in range(world):
                    assert bits_equal(outs[r], ring_want[r]), f"staged ring {what}, rank {r}: {mismatch_report(outs[r], ring_want[r])}"
        with pytest.raises(PcclError, match="may not exceed 1024"):
            eng.set_option("slot_threads", 1024); eng.set_option("slot_vecs", 4)
    finally:
        for key, val in (("slot_vecs", 0), ("slot_threads", 0), ("slot_lds_kib", 0), ("slot_store_waves", -1), ("num_blocks", 0), ("mode", "auto")):
            eng.set_option(key, val)


@pytest.mark.parametrize("world", [8, 24, 32])
def test_plans_that_mostly_write_take_larger_workgroups(engine_factory, world):
    """An allgather stores R times what it loads: up to 32 ranks it runs on the slot runner, with 256
    threads beyond 16 ranks (the register runner otherwise takes programs of that many ranks that
    read nothing back), and on 5 to 8 ranks with 1024 threads from 256 MiB per rank on.  An
    allreduce of the same ranks keeps the shape chosen from the rank count.  Results against the
    oracle at sizes with cut tiles, staged and in place."""
    n = world * (1000 + 37)
    jsons = graph_jsons("ring", "build_allgather", world, n, "float16", "sm", 1)
    chunk = n // world
    x = seeded_inputs("randn", world, chunk, "float16", seed=world)
    want = oracle_buffers(jsons, x, "float16", buffer_elems=n, place=lambda r: r * chunk)
    eng = engine_factory(world)
    for r, j in enumerate(jsons):
        eng.register_operation_json("ag", j, r)
    eng.set_option("phased", -1)                     # whatever PCCL_PHASED says: the automatic choice is what is tested
    shape = eng.get_option("slot_shape:ag")
    assert shape == ("256x2" if world == 8 else "256x1"), shape
    assert eng.get_option("runner_staged:ag") == "column_slot_kernel"
    outs = [torch.zeros(n, dtype=torch.float16, device="cuda") for _ in range(world)]
    eng.execute_operation("ag", [t.cuda() for t in x], outs)
    for r in range(world):
        assert bits_equal(outs[r], want[r]), f"staged, rank {r}: {mismatch_report(outs[r], want[r])}"
    bufs = []
    for r in range(world):
        b = torch.zeros(n, dtype=torch.float16)
        b[r * chunk:(r + 1) * chunk] = x[r]
        bufs.append(b.cuda())
    eng.execute_inplace("ag", bufs, sync=True)
    for r in range(world):
        assert bits_equal(bufs[r], want[r]), f"in place, rank {r}: {mismatch_report(bufs[r], want[r])}"
    # the same ranks, an allreduce: as many loads as stores
    ar = graph_jsons("ring", "build_allreduce", world, n, "float16", "sm", 1)
    for r, j in enumerate(ar):
        eng.register_operation_json("ar", j, r)
    assert eng.get_option("slot_shape:ar") == ("256x2" if world == 8 else "0x0")
    if world == 8:
        # the size from which 1024 threads pay is too large for the oracle: only the choice is checked here
        # (the full-size configuration tests run it)
        big = graph_jsons("ring", "build_allgather", world, 1 << 27, "float16", "sm", 1)
        for r, j in enumerate(big):
            eng.register_operation_json("ag_big", j, r)
        assert eng.get_option("slot_shape:ag_big") == "1024x1"
        eng16 = engine_factory(16)
        for r, j in enumerate(graph_jsons("ring", "build_allgather", 16, 1 << 25, "float16", "sm", 1)):
            eng16.register_operation_json("ag_big", j, r)
        assert eng16.get_option("slot_shape:ag_big") == "512x1"     # 16 ranks: from 64 MiB per rank on
        eng.set_option("slot_vecs", 2)                       # a shape that is asked for is kept
        try:
            assert eng.get_option("slot_shape:ag_big") == "256x2"
        finally:
            eng.set_option("slot_vecs", 0)


def test_slot_shape_options_are_checked_where_they_are_set(engine_factory):
    """A workgroup shape that the LDS cannot hold is refused by set_option itself, against the shape
    linking would choose with the other option left automatic, and the refused value is not kept:
    the next execution runs with the previous shape."""
    world, n = 16, 1 << 14
    jsons = graph_jsons("rhd", "build_allreduce", world, n, "float32", "sm", 1)
    x = seeded_inputs("randn", world, n, "float32", seed=4)
    want = oracle_buffers(jsons, x, "float32")
    eng = engine_factory(world)
    for r, j in enumerate(jsons):
        eng.register_operation_json("rhd", j, r)
    try:
        # 16 ranks: the automatic workgroup has 256 threads; 4 vectors per thread would need 256 KiB
        with pytest.raises(PcclError, match="KiB of LDS"):
            eng.set_option("slot_vecs", 4)
        assert eng.get_option("slot_vecs") == "0"
        eng.set_option("slot_threads", 64)
        eng.set_option("slot_vecs", 4)                      # 64 x 4 x 16 ranks x 16 B = 64 KiB: fine
        with pytest.raises(PcclError, match="KiB of LDS"):
            eng.set_option("slot_threads", 256)             # with the 4 vectors just set
        assert eng.get_option("slot_threads") == "64"
        with pytest.raises(PcclError, match="slot_direct=1"):
            eng.set_option("slot_direct", 0)                # fetching through registers takes one vector per thread
        assert eng.get_option("slot_direct") == "1"
        bufs = [t.cuda() for t in x]
        eng.execute_inplace("rhd", bufs, sync=True)
        for r in range(world):
            assert bits_equal(bufs[r], want[r]), mismatch_report(bufs[r], want[r])
        eng.set_option("slot_vecs", 1)
        eng.set_option("slot_direct", 0)
        with pytest.raises(PcclError, match="slot_direct=1"):
            eng.set_option("slot_vecs", 2)
    finally:
        for key, val in (("slot_direct", 1), ("slot_vecs", 0), ("slot_threads", 0)):
            eng.set_option(key, val)


@pytest.mark.parametrize("entry", ["inplace", "static"])
def test_launch_numbers_of_the_persistent_runner_wrap(engine_factory, entry):
    """Flags of the persistent runner hold the number of the launch that set them and are never
    cleared between launches; when the numbers run out the flags are cleared and the count restarts,
    on the host (eager launches) and on the device (launches recorded into a graph).  With both
    limits brought within reach, executions before, at and after each wrap give the oracle's bits."""
    import ctypes
    from pccl_amd import _lib
    world, n = 8, 1 << 15
    jsons = graph_jsons("ring", "build_allreduce", world, n, "bfloat16", "sm", 2)
    x = seeded_inputs("randn", world, n, "bfloat16", seed=31)
    want = oracle_buffers(jsons, x, "bfloat16")
    eng = engine_factory(world)
    name = f"wrap_{entry}"
    for r, j in enumerate(jsons):
        eng.register_operation_json(name, j, r)
    src = [t.cuda() for t in x]
    bufs = [t.clone() for t in src]
    L = _lib.lib()

    def execute(stream=None, sync=True):
        ptrs = (ctypes.c_void_p * world)(*[b.data_ptr() for b in bufs])
        s = stream if stream is not None else torch.cuda.current_stream().cuda_stream
        f = L.pccl_hip_execute_inplace if entry == "inplace" else L.pccl_hip_execute_inplace_static
        _lib.check(f(eng._h, name.encode(), ptrs, bufs[0].nbytes, s, 1 if sync else 0))

    eng.set_option("mode", "persistent")
    eng.set_option("test_host_epoch_limit", 5)
    eng.set_option("test_graph_epoch_limit", 0x40000000 + 4)
    try:
        for i in range(13):                                   # the host's numbers wrap at launches 6 and 11
            for b, t in zip(bufs, src):
                b.copy_(t)
            execute()
            for r in range(world):
                assert bits_equal(bufs[r], want[r]), f"eager launch {i}, rank {r}: {mismatch_report(bufs[r], want[r])}"
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.stream(side):
            with torch.cuda.graph(graph, stream=side):
                for b, t in zip(bufs, src):
                    b.copy_(t)
                execute(stream=side.cuda_stream, sync=False)
        torch.cuda.current_stream().wait_stream(side)
        for rep in range(9):                                  # the device's counter wraps at every fourth replay
            for b in bufs:
                b.zero_()
            torch.cuda.synchronize()
            graph.replay()
            torch.cuda.synchronize()
            for r in range(world):
                assert bits_equal(bufs[r], want[r]), f"replay {rep}, rank {r}: {mismatch_report(bufs[r], want[r])}"
            if rep % 3 == 2:                                  # eager launches between the replays
                for b, t in zip(bufs, src):
                    b.copy_(t)
                execute()
                for r in range(world):
                    assert bits_equal(bufs[r], want[r]), f"eager launch after replay {rep}, rank {r}"
        eng.sync_operation(name)
    finally:
        eng.set_option("test_host_epoch_limit", 0x40000000 - 16)
        eng.set_option("test_graph_epoch_limit", 0x7FFFFFF0)
        eng.set_option("mode", "auto")
