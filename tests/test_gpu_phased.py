"""The phased runner: chain plans (one accumulator per position, the result to a set of ranks) and
balanced trees on a persistent grid whose workgroups read together, meet, write together, meet.
Everything is compared with the CPU oracle bit for bit through the engine's C-ABI calls; the
meetings order nothing, so results must also be exact when they time out or are switched off."""
import pytest
import torch

from helpers import bits_equal, graph_jsons, mismatch_report, oracle_buffers, random_program, seeded_inputs

pytestmark = pytest.mark.gpu

CHUNK_VECS = 8192      # 16-byte vectors of every rank one workgroup takes per sweep (chain shapes)


def _register(eng, name, jsons):
    for r, j in enumerate(jsons):
        eng.register_operation_json(name, j, r)


def _check(got, want, what):
    for r, (g, w) in enumerate(zip(got, want)):
        assert bits_equal(g, w), f"{what}, rank {r}: {mismatch_report(g, w)}"


CASES = [
    # alg, method, world, elements, dtype, channels, extra, input kind, chain?, tree?
    ("ring", "build_allreduce", 8, 8 * 3 * 65536 + 8 * 24, "bfloat16", 4, {}, "randn", True, False),
    ("ring", "build_allreduce", 3, 3 * 100003, "float32", 1, {}, "randn", True, False),
    ("ring", "build_allreduce", 16, 16 * 40000, "float16", 2, {}, "randn", True, False),
    ("ring", "build_allreduce", 5, 5 * 77777, "float8_e4m3", 1, {}, "randn", True, False),
    ("tree", "build_allreduce", 32, 300007, "int32", 1, {"reduce_op": "sum"}, "randint", True, False),
    ("tree", "build_allreduce", 16, 250001, "float32", 1, {"reduce_op": "max"}, "randn", True, False),
    ("tree", "build_allreduce", 8, 131072 + 5, "bfloat16", 1, {"reduce_op": "min"}, "randn", True, False),
    ("rhd", "build_allreduce", 16, 16 * 50000, "int32", 1, {}, "randint", True, False),
    ("rhd", "build_allreduce", 16, 16 * 40960, "float32", 2, {}, "uniform", True, True),
    ("rhd", "build_allreduce", 8, 8 * 30000, "bfloat16", 1, {}, "randn", True, True),
    ("tree", "build_allreduce", 32, 200003, "float32", 1, {"reduce_op": "sum"}, "randn", True, True),
    ("tree", "build_allreduce", 64, 70001, "float16", 1, {"reduce_op": "sum"}, "randn0.1", True, True),
    ("tree", "build_allreduce", 2, 90001, "float32", 1, {"reduce_op": "sum"}, "randn", True, False),
]


@pytest.mark.parametrize("case", CASES, ids=lambda c: f"{c[0]}-R{c[2]}-{c[4]}-{c[6].get('reduce_op', 'sum')}")
def test_chain_and_tree_plans_in_place_and_staged(engine_factory, case):
    alg, method, world, n, dtype, channels, ext, kind, chain, tree = case
    jsons = graph_jsons(alg, method, world, n, dtype, "sm", channels, **ext)
    x = seeded_inputs(kind, world, n, dtype, seed=world + n % 97)
    want = oracle_buffers(jsons, x, dtype)
    eng = engine_factory(world)
    name = f"ph_{alg}_{world}_{dtype}_{ext.get('reduce_op', '')}"
    _register(eng, name, jsons)
    info = eng.op_info(name)
    assert (info["chain_segments"] == info["num_segments"]) == chain
    assert info["staged_chain_segments"] == info["chain_segments"]
    eng.set_option("phased", 1)
    try:
        # grids: one workgroup per CU; 5 workgroups (not a multiple of the XCD count, many sweeps and
        # meetings); meetings off; a wait that gives up at once
        for blocks, barriers, timeout in ((0, 1, 1000), (5, 1, 1000), (8, 0, 1000), (16, 1, 0)):
            # shapes: 512 x 16; 256 x 32 with each wave on 32 KiB in a row; the same read as slabs, the sums
            # changing hands through LDS before they are written (trees choose their shape themselves)
            # and 512 x 16 reading two sweeps before it writes their sums
            for shape, exchange, sweeps in (((-1, -1, -1),) if tree else ((0, 0, 1), (1, 0, 1), (1, 1, 1), (-1, -1, 2))):
                what = f"blocks={blocks} barriers={barriers} timeout={timeout} shape={shape} exchange={exchange} sweeps={sweeps}"
                print(f"{name}: {what}", flush=True)
                eng.set_option("num_blocks", blocks); eng.set_option("phased_barriers", barriers)
                eng.set_option("phased_timeout_us", timeout); eng.set_option("phased_shape", shape)
                eng.set_option("phased_exchange", exchange); eng.set_option("phased_sweeps", sweeps)
                bufs = [t.cuda() for t in x]
                eng.execute_inplace(name, bufs, sync=True)
                _check(bufs, want, f"in place, {what}")
                outs = eng.execute_operation(name, [t.cuda() for t in x])
                _check(outs, want, f"staged, {what}")
    finally:
        for key, val in (("phased", -1), ("num_blocks", 0), ("phased_barriers", 1), ("phased_timeout_us", 1000), ("phased_shape", -1),
                         ("phased_exchange", -1), ("phased_sweeps", -1)):
            eng.set_option(key, val)


@pytest.mark.parametrize("method", ["build_reduce_scatter", "build_allgather"])
def test_staged_reduce_scatter_and_allgather(engine_factory, method):
    """The staged plans of a ring reduce_scatter (eight ranks read, one written per chunk) and of an
    allgather (one read, eight written) are chains; in place a reduce_scatter leaves its partial sums
    in the other ranks and is not."""
    world, n = 8, 8 * (3 * CHUNK_VECS * 8 + 1000)     # fp16: 8 elements per vector; chunks cut by the chunk ends
    jsons = graph_jsons("ring", method, world, n, "float16", "sm", 1)
    chunk = n // world
    in_elems = n if method == "build_reduce_scatter" else chunk
    x = seeded_inputs("randn0.1", world, in_elems, "float16", seed=7)
    eng = engine_factory(world)
    name = "ph_" + method
    _register(eng, name, jsons)
    info = eng.op_info(name)
    assert info["staged_chain_segments"] == world
    assert info["chain_segments"] == (0 if method == "build_reduce_scatter" else world)
    # the staged call on the oracle: inputs placed in the rank buffers, the program, the output windows
    if method == "build_reduce_scatter":
        full = oracle_buffers(jsons, x, "float16")
        want = [full[r][r * chunk:(r + 1) * chunk] for r in range(world)]
    else:
        want = oracle_buffers(jsons, x, "float16", buffer_elems=n, place=lambda r: r * chunk)
        whole = torch.cat(x)
        for w in want:
            assert bits_equal(w, whole)
    eng.set_option("phased", 1)
    try:
        for blocks, sweeps in ((0, -1), (7, -1), (5, 1), (3, 2)):      # -1: two sweeps per write phase for the reduce_scatter
            eng.set_option("num_blocks", blocks); eng.set_option("phased_sweeps", sweeps)
            out_elems = chunk if method == "build_reduce_scatter" else n
            outs = [torch.empty(out_elems, dtype=torch.float16, device="cuda") for _ in range(world)]
            eng.execute_operation(name, [t.cuda() for t in x], outs)
            _check(outs, want, f"{method} blocks={blocks} sweeps={sweeps}")
    finally:
        eng.set_option("phased", -1); eng.set_option("num_blocks", 0); eng.set_option("phased_sweeps", -1)


def test_automatic_choice_and_what_is_not_a_chain(engine_factory):
    """Large chain plans go to the phased runner by themselves; a program that leaves different values
    in different ranks, or stores along the way, is not a chain plan and keeps running on the slot
    runner whatever the option says."""
    world = 8
    n = 4 * 256 * CHUNK_VECS * 8                         # bf16: 4 chunks per CU on a 256-CU GPU
    jsons = graph_jsons("ring", "build_allreduce", world, n, "bfloat16", "sm", 2)
    eng = engine_factory(world)
    _register(eng, "ph_auto", jsons)
    x = seeded_inputs("randn", world, n, "bfloat16", seed=3)
    want = oracle_buffers(jsons, x, "bfloat16")
    bufs = [t.cuda() for t in x]
    eng.execute_inplace("ph_auto", bufs, sync=True)
    _check(bufs, want, "automatic")
    rnd = random_program(4242, 4, 50000, 40, "float32", True)
    _register(eng4 := engine_factory(4), "ph_rnd", rnd)
    assert eng4.op_info("ph_rnd")["chain_segments"] == 0
    xr = seeded_inputs("randn", 4, 50000, "float32", seed=5)
    wr = oracle_buffers(rnd, xr, "float32")
    eng4.set_option("phased", 1)
    try:
        b = [t.cuda() for t in xr]
        eng4.execute_inplace("ph_rnd", b, sync=True)
        _check(b, wr, "not a chain plan")
    finally:
        eng4.set_option("phased", -1)


def test_more_workgroups_than_fit_at_once(engine_factory):
    """With more workgroups than the GPU holds at once a meeting cannot complete: the waits run out,
    the launch goes on unsynchronised and finishes with exact results, and the next launch meets
    normally again (the last workgroup to leave clears the meeting block)."""
    world, n = 8, 1200 * CHUNK_VECS * 8              # bf16: 1200 chunks of every rank
    jsons = graph_jsons("ring", "build_allreduce", world, n, "bfloat16", "sm", 1)
    x = seeded_inputs("randn", world, n, "bfloat16", seed=9)
    want = oracle_buffers(jsons, x, "bfloat16")
    eng = engine_factory(world)
    _register(eng, "ph_many", jsons)
    eng.set_option("phased", 1)
    try:
        for blocks, timeout in ((1100, 50), (0, 1000), (1100, 0), (0, 1000)):
            eng.set_option("num_blocks", blocks); eng.set_option("phased_timeout_us", timeout)
            bufs = [t.cuda() for t in x]
            eng.execute_inplace("ph_many", bufs, sync=True)
            _check(bufs, want, f"blocks={blocks} timeout={timeout}")
    finally:
        eng.set_option("phased", -1); eng.set_option("num_blocks", 0); eng.set_option("phased_timeout_us", 1000)


@pytest.mark.parametrize("case", [(4, "bfloat16", "sum", 1), (2, "float32", "max", 1), (8, "float16", "sum", 1), (2, "int32", "sum", 2), (3, "float32", "min", 1)])
def test_chunks_of_neighbouring_workgroups_interleaved(engine_factory, case):
    """Chains on up to 8 ranks whose segments are whole multiples of 128 chunks run with the chunks of
    128 neighbouring workgroups interleaved slab by slab (shape 5): in place and staged against the
    oracle, with the option that switches it off, and with a grid or a size that does not allow it."""
    world, dtype, op, channels = case
    es = 4 if dtype in ("float32", "int32") else 2
    seg_elems = 128 * CHUNK_VECS * (16 // es)                  # 16 MiB of every rank per segment
    n = world * channels * seg_elems
    jsons = graph_jsons("ring", "build_allreduce", world, n, dtype, "sm", channels, reduce_op=op)
    kind = "randint" if dtype == "int32" else "randn"
    x = seeded_inputs(kind, world, n, dtype, seed=17 + world)
    want = oracle_buffers(jsons, x, dtype)
    eng = engine_factory(world)
    _register(eng, "ph_lin", jsons)
    eng.set_option("phased", 1)
    try:
        assert eng.get_option("phased_shape_inplace:ph_lin") == "shape=5 group=128 meetings=1"
        assert eng.get_option("phased_shape_staged:ph_lin") == "shape=5 group=128 meetings=1"
        bufs = [t.cuda() for t in x]
        eng.execute_inplace("ph_lin", bufs, sync=True)
        _check(bufs, want, "interleaved, in place")
        outs = eng.execute_operation("ph_lin", [t.cuda() for t in x])
        _check(outs, want, "interleaved, staged")
        eng.set_option("phased_barriers", 0)
        bufs = [t.cuda() for t in x]
        eng.execute_inplace("ph_lin", bufs, sync=True)
        _check(bufs, want, "interleaved, no meetings")
        eng.set_option("phased_barriers", 1)
        eng.set_option("phased_linear", 0)
        assert eng.get_option("phased_shape_inplace:ph_lin").split()[0] in ("shape=0", "shape=4")     # 4 from two sweeps on
        bufs = [t.cuda() for t in x]
        eng.execute_inplace("ph_lin", bufs, sync=True)
        _check(bufs, want, "switched off")
        eng.set_option("phased_linear", -1)
        eng.set_option("num_blocks", 100)                       # a grid that 128 does not divide
        assert not eng.get_option("phased_shape_inplace:ph_lin").startswith("shape=5")
        bufs = [t.cuda() for t in x]
        eng.execute_inplace("ph_lin", bufs, sync=True)
        _check(bufs, want, "grid of 100")
        eng.set_option("num_blocks", 128)                       # one group per sweep
        assert eng.get_option("phased_shape_inplace:ph_lin") == "shape=5 group=128 meetings=1"
        bufs = [t.cuda() for t in x]
        eng.execute_inplace("ph_lin", bufs, sync=True)
        _check(bufs, want, "grid of 128")
        eng.set_option("num_blocks", 0)
    finally:
        eng.set_option("phased", -1); eng.set_option("phased_linear", -1); eng.set_option("num_blocks", 0); eng.set_option("phased_barriers", 1)
    # segments that are no multiple of 128 chunks keep the other shapes
    if world == 2:
        n2 = n + world * channels * CHUNK_VECS * (16 // es)
        eng2 = engine_factory(world)
        _register(eng2, "ph_lin2", graph_jsons("ring", "build_allreduce", world, n2, dtype, "sm", channels, reduce_op=op))
        eng2.set_option("phased", 1)
        assert not eng2.get_option("phased_shape_inplace:ph_lin2").startswith("shape=5")


@pytest.mark.parametrize("case", [(2, "float32", "sum", 1, 64), (4, "bfloat16", "sum", 2, 64), (8, "float16", "max", 1, 64),
                                  (2, "int32", "sum", 2, 64), (4, "float32", "min", 1, 32), (3, "bfloat16", "sum", 1, 128)])
def test_interleaved_groups_that_span_several_segments(engine_factory, case):
    """Segments of 64 chunks: a group of 128 workgroups spans two of them, and the rows of a thread
    belong to different segments with different source orders.  In place and staged against the
    oracle; segments of 32 chunks keep the other shapes (unless the plan mostly writes: the allgather
    test), and with three ranks of 128 chunks the plain interleaved kernel runs."""
    world, dtype, op, channels, seg_chunks = case
    es = 4 if dtype in ("float32", "int32") else 2
    n = world * channels * seg_chunks * CHUNK_VECS * (16 // es)
    jsons = graph_jsons("ring", "build_allreduce", world, n, dtype, "sm", channels, reduce_op=op)
    kind = "randint" if dtype == "int32" else "randn"
    x = seeded_inputs(kind, world, n, dtype, seed=31 + world + seg_chunks)
    want = oracle_buffers(jsons, x, dtype)
    eng = engine_factory(world)
    _register(eng, "ph_rows", jsons)
    eng.set_option("phased", 1)
    try:
        total = world * channels * seg_chunks
        how = eng.get_option("phased_shape_inplace:ph_rows")
        if total % 128 == 0 and seg_chunks >= 64:
            spans = 128 // seg_chunks
            assert how == ("shape=5 group=128 meetings=1" if spans == 1 else f"shape=5 group=128 segments={spans} meetings=1"), how
        else:
            assert not how.startswith("shape=5"), how
        bufs = [t.cuda() for t in x]
        eng.execute_inplace("ph_rows", bufs, sync=True)
        _check(bufs, want, f"in place ({how})")
        outs = eng.execute_operation("ph_rows", [t.cuda() for t in x])
        _check(outs, want, f"staged ({how})")
        eng.set_option("num_blocks", 128)
        bufs = [t.cuda() for t in x]
        eng.execute_inplace("ph_rows", bufs, sync=True)
        _check(bufs, want, "grid of 128")
    finally:
        eng.set_option("phased", -1); eng.set_option("num_blocks", 0)


def test_allgather_on_interleaved_chunks(engine_factory):
    """A plan that mostly writes stays on the slot runner unless its chunks can be interleaved: an
    allgather of 16 MiB pieces goes to the phased runner's shape 5 by itself (staged and in place),
    one of 8 MiB pieces does not.  Against the oracle; an allgather only copies."""
    world, dtype = 4, "float16"
    chunk = 128 * CHUNK_VECS * 8                               # 16 MiB of fp16 per rank's piece
    n = world * chunk
    jsons = graph_jsons("ring", "build_allgather", world, n, dtype, "sm", 1)
    x = seeded_inputs("randn", world, chunk, dtype, seed=5)
    want = oracle_buffers(jsons, x, dtype, buffer_elems=n, place=lambda r: r * chunk)
    eng = engine_factory(world)
    _register(eng, "ag_lin", jsons)
    eng.set_option("phased", -1)                               # the automatic choice, whatever PCCL_PHASED says
    assert eng.get_option("runner_staged:ag_lin") == "phased_kernel"
    assert eng.get_option("phased_shape_staged:ag_lin") == "shape=5 group=128 meetings=1"
    outs = [torch.zeros(n, dtype=torch.float16, device="cuda") for _ in range(world)]
    eng.execute_operation("ag_lin", [t.cuda() for t in x], outs)
    _check(outs, want, "staged")
    bufs = []
    for r in range(world):
        b = torch.zeros(n, dtype=torch.float16)
        b[r * chunk:(r + 1) * chunk] = x[r]
        bufs.append(b.cuda())
    assert eng.get_option("phased_shape_inplace:ag_lin") == "shape=5 group=128 meetings=1"
    eng.execute_inplace("ag_lin", bufs, sync=True)
    _check(bufs, want, "in place")
    eng.set_option("phased_linear", 0)
    assert eng.get_option("runner_staged:ag_lin") == "column_slot_kernel"
    eng.set_option("phased_linear", -1)
    # pieces of 8 MiB (64 chunks): a group spans two of them
    half = graph_jsons("ring", "build_allgather", world, n // 2, dtype, "sm", 1)
    _register(eng, "ag_half", half)
    assert eng.get_option("phased_shape_staged:ag_half") == "shape=5 group=128 segments=2 meetings=1"
    xh = seeded_inputs("randn", world, chunk // 2, dtype, seed=6)
    wanth = oracle_buffers(half, xh, dtype, buffer_elems=n // 2, place=lambda r: r * (chunk // 2))
    outs = [torch.zeros(n // 2, dtype=torch.float16, device="cuda") for _ in range(world)]
    eng.execute_operation("ag_half", [t.cuda() for t in xh], outs)
    _check(outs, wanth, "two segments per group, staged")
    # pieces of 4 MiB (32 chunks): four segments per group, for a plan that mostly writes
    quarter = graph_jsons("ring", "build_allgather", world, n // 4, dtype, "sm", 1)
    _register(eng, "ag_quarter", quarter)
    assert eng.get_option("phased_shape_staged:ag_quarter") == "shape=5 group=128 segments=4 meetings=1"
    xq = seeded_inputs("randn", world, chunk // 4, dtype, seed=7)
    wantq = oracle_buffers(quarter, xq, dtype, buffer_elems=n // 4, place=lambda r: r * (chunk // 4))
    outs = [torch.zeros(n // 4, dtype=torch.float16, device="cuda") for _ in range(world)]
    eng.execute_operation("ag_quarter", [t.cuda() for t in xq], outs)
    _check(outs, wantq, "four segments per group, staged")
    # pieces of 1 MiB: too small for any of it, the slot runner
    tiny = graph_jsons("ring", "build_allgather", world, n // 16, dtype, "sm", 1)
    _register(eng, "ag_tiny", tiny)
    assert eng.get_option("runner_staged:ag_tiny") == "column_slot_kernel"
    assert eng.get_option("phased_shape_staged:ag_tiny") == "none"


def test_two_launches_of_one_operation_on_two_streams(engine_factory):
    """In-place calls on different tensors may overlap on the GPU.  Two phased launches of one
    operation then share its meeting block and lose their phases, which costs time and nothing else:
    both results are exact, and the next launch on its own meets normally again."""
    world, n = 8, 600 * CHUNK_VECS * 8                # bf16: 600 chunks of every rank, more than two sweeps
    jsons = graph_jsons("ring", "build_allreduce", world, n, "bfloat16", "sm", 1)
    xa = seeded_inputs("randn", world, n, "bfloat16", seed=21)
    xb = seeded_inputs("randn", world, n, "bfloat16", seed=22)
    want_a, want_b = oracle_buffers(jsons, xa, "bfloat16"), oracle_buffers(jsons, xb, "bfloat16")
    eng = engine_factory(world)
    _register(eng, "ph_two", jsons)
    eng.set_option("phased", 1)
    try:
        a = [t.cuda() for t in xa]
        eng.execute_inplace("ph_two", a, sync=True)          # linked and uploaded
        _check(a, want_a, "alone")
        s1, s2 = torch.cuda.Stream(), torch.cuda.Stream()
        for rep in range(3):
            a, b = [t.cuda() for t in xa], [t.cuda() for t in xb]
            torch.cuda.synchronize()
            with torch.cuda.stream(s1):
                eng.execute_inplace("ph_two", a)
            with torch.cuda.stream(s2):
                eng.execute_inplace("ph_two", b)
            torch.cuda.synchronize()
            _check(a, want_a, f"first of two, repetition {rep}")
            _check(b, want_b, f"second of two, repetition {rep}")
        a = [t.cuda() for t in xa]
        eng.execute_inplace("ph_two", a, sync=True)
        _check(a, want_a, "alone again")
    finally:
        eng.set_option("phased", -1)


@pytest.mark.parametrize("sweeps", [1, 2])
def test_phased_launches_recorded_into_a_graph(engine_factory, sweeps):
    """A phased launch is one kernel and needs no set-up per launch (the meeting block cleans itself),
    so it can be recorded and replayed, with one sweep per write phase or two; every replay against
    the oracle, eager work in between."""
    world, n = 8, 16 * CHUNK_VECS * 8                  # 16 chunks
    jsons = graph_jsons("ring", "build_allreduce", world, n, "bfloat16", "sm", 2)
    x = seeded_inputs("randn", world, n, "bfloat16", seed=13)
    want = oracle_buffers(jsons, x, "bfloat16")
    eng = engine_factory(world)
    _register(eng, "ph_graph", jsons)
    eng.set_option("phased", 1)
    eng.set_option("phased_sweeps", sweeps)
    eng.set_option("num_blocks", 5)                    # four sweeps of five workgroups: meetings inside the recorded launch
    try:
        src = [t.cuda() for t in x]
        bufs = [t.clone() for t in src]
        eng.execute_inplace("ph_graph", bufs, sync=True)
        _check(bufs, want, "eager")
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.stream(side):
            with torch.cuda.graph(graph, stream=side):
                for b, t in zip(bufs, src):
                    b.copy_(t)
                eng.execute_inplace("ph_graph", bufs)
        torch.cuda.current_stream().wait_stream(side)
        for rep in range(4):
            for b in bufs:
                b.fill_(float(rep))
            torch.cuda.synchronize()
            graph.replay()
            torch.cuda.synchronize()
            _check(bufs, want, f"replay {rep}")
    finally:
        eng.set_option("phased", -1); eng.set_option("phased_sweeps", -1); eng.set_option("num_blocks", 0)


SPECIAL_BITS = {   # quiet NaNs with payloads, a signalling NaN, infinities, zeros, the smallest denormal, the largest finite values
    "float32": [0x7FC00000, 0x7FC12345, 0xFFC00001, 0x7F800001, 0x7F800000, 0xFF800000, 0x00000000, 0x80000000, 0x00000001, 0x7F7FFFFF, 0xFF7FFFFF],
    "bfloat16": [0x7FC0, 0x7FC5, 0xFFC1, 0x7F81, 0x7F80, 0xFF80, 0x0000, 0x8000, 0x0001, 0x7F7F, 0xFF7F],
    "float16": [0x7E00, 0x7E05, 0xFE01, 0x7C01, 0x7C00, 0xFC00, 0x0000, 0x8000, 0x0001, 0x7BFF, 0xFBFF],
}


def _with_specials(x, dtype, seed):
    """One element in a hundred of every rank replaced by a special bit pattern."""
    import numpy as np
    from helpers import from_raw, to_raw
    rng = np.random.default_rng(seed)
    out = []
    for t in x:
        raw = to_raw(t).copy()
        where = rng.random(raw.shape[0]) < 0.01
        raw[where] = rng.choice(np.array(SPECIAL_BITS[dtype], dtype=raw.dtype), int(where.sum()))
        out.append(from_raw(raw, dtype))
    return out


@pytest.mark.parametrize("case", [
    ("ring", "build_allreduce", 8, "bfloat16", "sum"), ("ring", "build_allreduce", 4, "float16", "sum"),
    ("ring", "build_allreduce", 16, "float32", "sum"), ("tree", "build_allreduce", 16, "float32", "max"),
    ("tree", "build_allreduce", 8, "float16", "min"), ("tree", "build_allreduce", 32, "bfloat16", "max"),
    ("rhd", "build_allreduce", 16, "float32", "sum"), ("tree", "build_allreduce", 32, "bfloat16", "sum"),
    ("rhd", "build_allreduce", 8, "float16", "sum"), ("ring", "build_allgather", 8, "float32", "sum"),
], ids=lambda c: f"{c[0]}-{c[1][6:]}-R{c[2]}-{c[3]}-{c[4]}")
def test_nans_infinities_and_zeros_through_chains_and_trees(engine_factory, case):
    """The read phases canonicalise NaN results once, at the end of a chain or tree, instead of after
    every step: same bits as the oracle, which does it step by step - NaN payloads and signalling
    NaNs among the inputs, infinities of both signs meeting in a sum, signed zeros under MAX and MIN.
    An allgather only copies: its NaNs keep their payloads."""
    alg, method, world, dtype, op = case
    per = {"float32": 4, "bfloat16": 8, "float16": 8}[dtype]
    n = world * (2 * CHUNK_VECS * per + 40)              # chunks cut by the ends, for the vector-by-vector path too
    ext = {} if method == "build_allgather" else {"reduce_op": op}
    jsons = graph_jsons(alg, method, world, n, dtype, "sm", 1, **ext)
    gather = method == "build_allgather"
    chunk = n // world
    x = _with_specials(seeded_inputs("randn", world, chunk if gather else n, dtype, seed=world), dtype, seed=17 + world)
    want = oracle_buffers(jsons, x, dtype, buffer_elems=n, place=(lambda r: r * chunk) if gather else None)
    eng = engine_factory(world)
    name = f"nan_{alg}_{method}_{world}_{dtype}_{op}"
    _register(eng, name, jsons)
    assert eng.op_info(name)["chain_segments" if not gather else "staged_chain_segments"] > 0
    eng.set_option("phased", 1)
    try:
        for exchange, sweeps in ((0, -1), (1, -1), (-1, 2)):
            eng.set_option("phased_exchange", exchange); eng.set_option("phased_sweeps", sweeps)
            if gather:
                outs = [torch.empty(n, dtype=x[0].dtype, device="cuda") for _ in range(world)]
                eng.execute_operation(name, [t.cuda() for t in x], outs)
                _check(outs, want, f"staged, exchange={exchange}")
            else:
                bufs = [t.cuda() for t in x]
                eng.execute_inplace(name, bufs, sync=True)
                _check(bufs, want, f"in place, exchange={exchange}")
                assert eng.get_option(f"runner_inplace:{name}") == "phased_kernel"
    finally:
        eng.set_option("phased", -1); eng.set_option("phased_exchange", -1); eng.set_option("phased_sweeps", -1)
