"""The benchmark configurations at their full sizes, checked through size-independent properties
evaluated with plain torch on the GPU (the CPU oracle covers the same graphs at small sizes in
test_gpu_parity.py):

* ring / RHD / tree results must equal the schedule's per-element reduction order written with
  torch adds in the storage dtype (bit-exact), and all ranks must hold identical bits;
* int32 SUM and float MAX must equal torch.stack(x).sum(0) / .amax(0) (order-insensitive);
* reduce_scatter and allgather must satisfy their definitions chunk by chunk.
"""
import pytest
import torch

from helpers import TORCH_DTYPE, graph_jsons
from pccl_amd.dsl import ragged_cuts

pytestmark = pytest.mark.gpu


def dev_inputs(kind, world, n, dtype, seed=0):
    """Seeded inputs generated on the GPU (full-size inputs from the CPU generator take minutes)."""
    g = torch.Generator(device="cuda").manual_seed(seed)
    outs = []
    for _ in range(world):
        if kind == "randn":
            x = torch.randn(n, generator=g, device="cuda")
        elif kind == "uniform":
            x = torch.rand(n, generator=g, device="cuda") * 2 - 1
        elif kind == "randn0.1":
            x = torch.randn(n, generator=g, device="cuda") * 0.1
        else:
            x = torch.randint(-1000, 1000, (n,), generator=g, device="cuda")
        outs.append(x.to(TORCH_DTYPE[dtype]))
    return outs


def same_bits(a, b):
    if a.dtype in (torch.float16, torch.bfloat16):
        return torch.equal(a.view(torch.int16), b.view(torch.int16))
    if a.dtype == torch.float32:
        return torch.equal(a.view(torch.int32), b.view(torch.int32))
    return torch.equal(a, b)


def register(engine, name, jsons, mode):
    for r, j in enumerate(jsons):
        engine.register_operation_json(name, j, r)
    engine.set_option("mode", mode)


def rhd_expected(x, world, lo, n):
    v = [t[lo:lo + n].clone() for t in x]
    k = 1
    while k < world:
        v = [v[r ^ k] + v[r] for r in range(world)]
        k <<= 1
    return v[0]


@pytest.mark.parametrize("mode", ["column", "stepwise", "persistent"])
def test_config3_rhd_16_ranks_64mb_f32_two_channels(engine_factory, mode):
    world, n = 16, 16_777_216
    print(f"config 3: RHD R={world} n={n} f32 2 channels, mode={mode}", flush=True)
    jsons = graph_jsons("rhd", "build_allreduce", world, n, "float32", "sm", 2)
    x = dev_inputs("uniform", world, n, "float32")
    engine = engine_factory(world)
    register(engine, f"c3_{mode}", jsons, mode)
    bufs = [t.clone() for t in x]
    engine.execute_inplace(f"c3_{mode}", bufs, sync=True)
    want = rhd_expected(x, world, 0, n)
    assert same_bits(bufs[0], want)
    for r in range(1, world):
        assert same_bits(bufs[r], bufs[0]), f"rank {r} differs from rank 0"
    exact = sum(t.double() for t in x)
    assert torch.all((bufs[0].double() - exact).abs() <= 1e-6 * world * exact.abs().clamp_min(1.0))
    info = engine.op_info(f"c3_{mode}")
    assert info["algorithmic_bytes"] == 75 * n * 4        # 5 (1 - 1/R) R S


@pytest.mark.parametrize("mode", ["column", "stepwise", "persistent"])
@pytest.mark.parametrize("dtype,redop,kind", [("int32", "sum", "randint"), ("float32", "max", "randn")])
def test_config5_tree_32_ranks_96mb_ragged(engine_factory, dtype, redop, kind, mode):
    world, n = 32, 25_165_824
    print(f"config 5: tree R={world} n={n} {dtype} {redop} ragged, mode={mode}", flush=True)
    cuts = ragged_cuts(n, 8, seed=0)
    assert all(c % 4 for c in cuts)
    jsons = graph_jsons("tree", "build_allreduce", world, n, dtype, "sm", 1, reduce_op=redop, cuts=cuts)
    x = dev_inputs(kind, world, n, dtype)
    engine = engine_factory(world)
    name = f"c5_{dtype}_{mode}"
    register(engine, name, jsons, mode)
    bufs = [t.clone() for t in x]
    engine.execute_inplace(name, bufs, sync=True)
    if redop == "sum":
        want = x[0].clone()
        for t in x[1:]:
            want += t                                    # int32 wraps; any order gives the same bits
    else:
        want = torch.stack(x).amax(0)
    for r in range(world):
        assert same_bits(bufs[r], want), f"rank {r}"
    info = engine.op_info(name)
    assert info["algorithmic_bytes"] == 155 * n * 4      # 5 (R-1) S
    assert info["num_data_ops"] == 62 * 8                # every tree op cut into 8 ragged pieces


C4_SIZES = [4096 * 4 ** k for k in range(9)] + [512 << 20]      # 4 KB .. 256 MB in powers of 4, and 512 MB


@pytest.mark.parametrize("mode", ["column", "stepwise", "persistent"])
@pytest.mark.parametrize("nbytes", C4_SIZES)
def test_config4_reduce_scatter_allgather_fp16(engine_factory, nbytes, mode):
    """Configuration 4: every size of the sweep in every mode, as staged calls.  The results must
    equal the ring's reduction order written with torch fp16 adds and the definitions of the two
    collectives; up to 16 MB per rank they are also compared with the CPU oracle."""
    from helpers import bits_equal, oracle_buffers
    world = 8
    n = nbytes // 2
    chunk = n // world
    print(f"config 4: RS/AG R={world} {nbytes} B per rank fp16, mode={mode}", flush=True)
    engine = engine_factory(world)
    x = dev_inputs("randn0.1", world, n, "float16")
    with_oracle = nbytes <= (16 << 20)
    # reduce_scatter: chunk r of the ring-ordered sum lands on rank r
    name = f"rs_{nbytes}_{mode}"
    jsons = graph_jsons("ring", "build_reduce_scatter", world, n, "float16", "sm", 1)
    register(engine, name, jsons, mode)
    outs = engine.execute_operation(name, x, [torch.zeros(chunk, dtype=torch.float16, device="cuda") for _ in range(world)])
    for c in range(world):
        lo = c * chunk
        # chunk c travels c+1 -> c+2 -> ... -> c: acc = x_{c+1}; acc = x_{c+1+k} + acc
        acc = x[(c + 1) % world][lo:lo + chunk].clone()
        for k in range(1, world):
            acc = x[(c + 1 + k) % world][lo:lo + chunk] + acc
        assert same_bits(outs[c], acc), f"reduce_scatter chunk {c}"
    if with_oracle:
        want = oracle_buffers(jsons, [t.cpu() for t in x], "float16")
        for c in range(world):
            assert bits_equal(outs[c], want[c][c * chunk:(c + 1) * chunk]), f"reduce_scatter chunk {c} against the oracle"
    del outs
    # allgather: rank r contributes chunk r
    name = f"ag_{nbytes}_{mode}"
    jsons = graph_jsons("ring", "build_allgather", world, n, "float16", "sm", 1)
    register(engine, name, jsons, mode)
    parts = [t[:chunk].contiguous() for t in x]
    outs = engine.execute_operation(name, parts, [torch.zeros(n, dtype=torch.float16, device="cuda") for _ in range(world)])
    whole = torch.cat(parts)
    for r in range(world):
        assert same_bits(outs[r], whole), f"allgather rank {r}"
    if with_oracle:
        want = oracle_buffers(jsons, [p.cpu() for p in parts], "float16", buffer_elems=n, place=lambda r: r * chunk)
        for r in range(world):
            assert bits_equal(outs[r], want[r]), f"allgather rank {r} against the oracle"
    engine.set_option("mode", "auto")


@pytest.mark.parametrize("dtype,redop,kind", [("int32", "sum", "randint"), ("float32", "max", "randn")])
def test_config5_through_the_superoptimising_compiler(engine_factory, dtype, redop, kind):
    """Configuration 5's graphs as `Compiler(enable_superopt=True)` emits them: the data ops arrive as
    tma.reduce / tma.copy under the executor cuda_tma (the upgrade the reference's pass makes,
    pccl/dsl/superopt/pass_.py:76-87) and run as the SM ops, at the full size, ragged pieces and all."""
    import json
    from pccl_amd.dsl import ALGORITHMS, Compiler
    world, n = 32, 25_165_824
    print(f"config 5 through Compiler(enable_superopt=True): tree R={world} n={n} {dtype} {redop}", flush=True)
    cuts = ragged_cuts(n, 8, seed=0)
    tree = ALGORITHMS["tree"]()
    comp = Compiler(enable_superopt=True, topology=None)
    docs = [comp.compile_to_dict(tree.build_allreduce(r, world, n, dtype=dtype, executor="sm", num_channels=1,
                                                      reduce_op=redop, cuts=cuts)) for r in range(world)]
    prims = {op["primitive"] for d in docs for op in d["operations"]}
    execs = {op["executor"] for d in docs for op in d["operations"] if op["primitive"].startswith(("tma.", "sm."))}
    assert {"tma.reduce", "tma.copy"} <= prims and "sm.reduce" not in prims and "sm.copy" not in prims
    assert execs == {"cuda_tma"}
    x = dev_inputs(kind, world, n, dtype)
    engine = engine_factory(world)
    want = torch.stack(x).sum(0, dtype=torch.int32) if redop == "sum" else torch.stack(x).amax(0)
    for mode in ("auto", "persistent"):
        name = f"c5_superopt_{dtype}_{mode}"
        register(engine, name, [json.dumps(d) for d in docs], mode)
        bufs = [t.clone() for t in x]
        engine.execute_inplace(name, bufs, sync=True)
        for r in range(world):
            assert same_bits(bufs[r], want), f"mode {mode}, rank {r}"
        del bufs
    engine.set_option("mode", "auto")


def test_config2_prescribed_inputs_match_the_committed_oracle_hash_in_every_mode(engine_factory):
    """The headline configuration on its prescribed inputs (CPU generator, seed 0, drawn rank by rank
    in eight slices and cast to bf16): the result of the column, level and persistent runners must
    hash to what the CPU oracle produced for the full graph (tests/golden/headline_sha256.json,
    written by tests/golden/make_headline_sha256.py)."""
    import hashlib
    import json
    import os
    from helpers import GOLDEN
    golden = json.load(open(os.path.join(GOLDEN, "headline_sha256.json")))
    world, n, slices = 8, 268_435_456, 8
    print("config 2 on the prescribed inputs against the committed sha256, three modes", flush=True)

    def sha(t):
        h = hashlib.sha256()
        flat = t.view(torch.int16)
        for i in range(0, flat.numel(), 1 << 26):
            h.update(flat[i:i + (1 << 26)].cpu().numpy().tobytes())
        return h.hexdigest()

    g = torch.Generator().manual_seed(0)
    per = n // slices
    x = []
    for r in range(world):
        buf = torch.empty(n, dtype=torch.bfloat16, device="cuda")
        for s in range(slices):
            buf[s * per:(s + 1) * per] = torch.randn(per, generator=g).to(torch.bfloat16).cuda()
        x.append(buf)
        print(f"  rank {r} drawn", flush=True)
    assert sha(x[0]) == golden["input_sha256_per_rank"][0] and sha(x[7]) == golden["input_sha256_per_rank"][7]
    jsons = graph_jsons("ring", "build_allreduce", world, n, "bfloat16", "sm", 4)
    engine = engine_factory(world)
    for mode in ("column", "stepwise", "persistent"):
        print(f"  mode={mode}", flush=True)
        register(engine, f"c2_golden_{mode}", jsons, mode)
        bufs = [t.clone() for t in x]
        engine.execute_inplace(f"c2_golden_{mode}", bufs, sync=True)
        assert sha(bufs[0]) == golden["output_sha256"], f"mode {mode}"
        for r in range(1, world):
            assert same_bits(bufs[r], bufs[0]), f"mode {mode}: rank {r} differs from rank 0"
        del bufs
    engine.set_option("mode", "auto")


def test_config2_headline_shape_in_all_modes_agree(engine_factory):
    """512 MiB per rank, bf16, 4 channels: the column, level and persistent runners must produce the
    same bits."""
    world, n = 8, 268_435_456
    print("config 2: ring R=8 512 MiB bf16 4 channels, column vs stepwise vs persistent", flush=True)
    jsons = graph_jsons("ring", "build_allreduce", world, n, "bfloat16", "sm", 4)
    x = dev_inputs("randn", world, n, "bfloat16")
    engine = engine_factory(world)
    results = {}
    for mode in ("column", "stepwise", "persistent"):
        register(engine, f"c2_{mode}", jsons, mode)
        bufs = [t.clone() for t in x]
        engine.execute_inplace(f"c2_{mode}", bufs, sync=True)
        for r in range(1, world):
            assert same_bits(bufs[r], bufs[0])
        results[mode] = bufs[0]
        del bufs
    assert same_bits(results["column"], results["stepwise"])
    assert same_bits(results["column"], results["persistent"])
    per_ch, per_rank = n // 4, n // 32
    for ch in (0, 3):
        for c in (0, 5):
            lo = ch * per_ch + c * per_rank
            acc = x[c][lo:lo + per_rank].clone()
            for k in range(1, world):
                acc = x[(c + k) % world][lo:lo + per_rank] + acc
            assert same_bits(results["column"][lo:lo + per_rank], acc)


def test_largest_rank_buffers_the_graph_format_allows(engine_factory):
    """Offsets and sizes in a graph are 32-bit element counts (reference include/engine/fused_step.h:11-14),
    so the largest rank buffer is 2^31 - 1 elements.  A two-rank f32 ring on 2^31 - 2 elements (8 GiB per
    rank, chunks of 2^30 - 1 elements, so the second chunk starts 4 bytes short of 4 GiB and off 16-byte
    alignment) puts byte offsets beyond 2^32 through every runner.  Integer-valued inputs make the sum
    exact, and with two ranks the order of the one addition does not matter."""
    world, n = 2, (1 << 31) - 2
    print(f"largest buffers: ring R={world} n={n} f32, column / stepwise / persistent / staged", flush=True)
    jsons = graph_jsons("ring", "build_allreduce", world, n, "float32", "sm", 1)
    x = dev_inputs("randint", world, n, "float32")
    want = x[0] + x[1]
    engine = engine_factory(world)
    for mode in ("column", "stepwise", "persistent"):
        print(f"  mode={mode}", flush=True)
        register(engine, f"big_{mode}", jsons, mode)
        bufs = [t.clone() for t in x]
        engine.execute_inplace(f"big_{mode}", bufs, sync=True)
        for r in range(world):
            assert same_bits(bufs[r], want), f"mode {mode}, rank {r}"
        del bufs
    print("  staged call", flush=True)
    register(engine, "big_staged", jsons, "auto")
    outs = [torch.full((n,), -1.0, device="cuda") for _ in range(world)]
    engine.execute_operation("big_staged", x, outs)
    for r in range(world):
        assert same_bits(outs[r], want), f"staged call, rank {r}"
    assert engine.op_info("big_staged")["algorithmic_bytes"] == 5 * n * 4


def test_config3_full_size_against_the_cpu_oracle(engine_factory):
    """Configuration 3 at its full size (16 x 64 MiB f32, two channels) with the prescribed inputs
    from the CPU generator, the GPU result compared bit for bit with the CPU oracle's (about a
    gigabyte of buffers; the oracle needs a few seconds for it)."""
    from helpers import bits_equal, oracle_buffers, seeded_inputs
    world, n = 16, 16_777_216
    print("config 3 at full size against the oracle", flush=True)
    jsons = graph_jsons("rhd", "build_allreduce", world, n, "float32", "sm", 2)
    x = seeded_inputs("uniform", world, n, "float32", seed=0)
    want = oracle_buffers(jsons, x, "float32")
    engine = engine_factory(world)
    register(engine, "c3_oracle", jsons, "auto")
    bufs = [t.cuda() for t in x]
    engine.execute_inplace("c3_oracle", bufs, sync=True)
    for r in range(world):
        assert bits_equal(bufs[r], want[r]), f"rank {r}"


@pytest.mark.parametrize("runner", ["phased", "slot", "stepwise", "persistent"])
def test_rank_buffers_larger_than_4_gib(engine_factory, runner):
    """Byte offsets inside a rank buffer pass 2^32 (element offsets stay below the 2^31 of the trigger
    layout): a 2-rank f32 ring allreduce on 5 GiB per rank, in place, on every runner.  Both ranks must
    hold x0 + x1, which is the same bits in either order, over the whole buffer including its last
    vectors; a staged reduce_scatter of the same size checks the far end of the input windows."""
    world, n = 2, 1_342_177_280 + 12                       # 5 GiB and three vectors
    x = dev_inputs("randn", world, n, "float32", seed=11)
    want = x[0] + x[1]
    eng = engine_factory(world)
    jsons = graph_jsons("ring", "build_allreduce", world, n, "float32", "sm", 1)
    register(eng, "big", jsons, {"phased": "column", "slot": "column"}.get(runner, runner))
    eng.set_option("phased", 1 if runner == "phased" else 0)
    try:
        bufs = [t.clone() for t in x]
        print(f"{runner}: in place, {n} elements per rank", flush=True)
        eng.execute_inplace("big", bufs, sync=True)
        if runner in ("phased", "slot"):
            assert eng.get_option("runner_inplace:big") == ("phased_kernel" if runner == "phased" else "column_slot_kernel")
        for r in range(world):
            assert same_bits(bufs[r], want), f"rank {r}"
        del bufs
        rs = graph_jsons("ring", "build_reduce_scatter", world, n, "float32", "sm", 1)
        for r, j in enumerate(rs):
            eng.register_operation_json("big_rs", j, r)
        chunk = n // world
        outs = [torch.empty(chunk, dtype=torch.float32, device="cuda") for _ in range(world)]
        print(f"{runner}: staged reduce_scatter", flush=True)
        eng.execute_operation("big_rs", x, outs)
        for r in range(world):
            assert same_bits(outs[r], want[r * chunk:(r + 1) * chunk]), f"reduce_scatter rank {r}"
    finally:
        eng.set_option("mode", "auto"); eng.set_option("phased", -1)
        del x, want
        torch.cuda.empty_cache()
