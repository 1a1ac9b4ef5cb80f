"""Pins for the CPU oracle (oracle/pccl_oracle.c).  None of these tests re-type the oracle's own
formulas: every check is against an independent authority — torch / numpy arithmetic, the closed
forms of the reference's correctness script, or a brute-force evaluation of a schedule's
per-element reduction order written directly from the schedule definitions.
"""
import json

import numpy as np
import pytest
import torch

from helpers import (FP8_MAX, TORCH_DTYPE, bits_equal, carry_expected, carry_ops, from_raw, graph_jsons, mismatch_report,
                     oracle, oracle_buffers, seeded_inputs, to_raw)


# ------------------------------------------------------------------------------- element arithmetic

def _pairs_f16():
    """A dense sample of half-precision pairs: every exponent, both signs, subnormals, specials."""
    rng = np.random.default_rng(0)
    a = rng.integers(0, 1 << 16, 1 << 20, dtype=np.uint16)
    b = rng.integers(0, 1 << 16, 1 << 20, dtype=np.uint16)
    edge = np.array([0x0000, 0x8000, 0x0001, 0x8001, 0x03FF, 0x0400, 0x7BFF, 0xFBFF, 0x7C00, 0xFC00,
                     0x3C00, 0xBC00, 0x7BFE, 0x0002, 0x3555, 0x7A00], dtype=np.uint16)
    ea, eb = np.meshgrid(edge, edge)
    return np.concatenate([a, ea.ravel()]), np.concatenate([b, eb.ravel()])


def _canon_nan_equal(got_bits, want_bits, nan_mask, canon):
    """Equal everywhere; where the true result is NaN the oracle must give the canonical NaN."""
    ok = np.where(nan_mask, got_bits == canon, got_bits == want_bits)
    return bool(ok.all()), int((~ok).sum())


def test_f16_add_matches_numpy_and_torch():
    a, b = _pairs_f16()
    got = oracle.reduce("float16", "sum", a, b)
    with np.errstate(all="ignore"):
        want = (a.view(np.float16) + b.view(np.float16))          # numpy: float add, one rounding
    nan = np.isnan(want)
    ok, bad = _canon_nan_equal(got, want.view(np.uint16), nan, 0x7FFF)
    assert ok, f"{bad} mismatches vs numpy float16"
    t = (torch.from_numpy(a.view(np.int16)).view(torch.float16) + torch.from_numpy(b.view(np.int16)).view(torch.float16))
    ok, bad = _canon_nan_equal(got, t.view(torch.int16).numpy().view(np.uint16), nan, 0x7FFF)
    assert ok, f"{bad} mismatches vs torch float16"


def test_bf16_add_matches_torch():
    rng = np.random.default_rng(1)
    a = rng.integers(0, 1 << 16, 1 << 20, dtype=np.uint16)
    b = rng.integers(0, 1 << 16, 1 << 20, dtype=np.uint16)
    got = oracle.reduce("bfloat16", "sum", a, b)
    ta = torch.from_numpy(a.view(np.int16)).view(torch.bfloat16)
    tb = torch.from_numpy(b.view(np.int16)).view(torch.bfloat16)
    want = (ta + tb)
    nan = torch.isnan(want).numpy()
    ok, bad = _canon_nan_equal(got, want.view(torch.int16).numpy().view(np.uint16), nan, 0x7FFF)
    assert ok, f"{bad} mismatches vs torch bfloat16"
    # and against the definition: round-to-nearest-even of the exact sum (float64 is exact here)
    exact = ta.double() + tb.double()
    want2 = exact.to(torch.bfloat16)
    ok, bad = _canon_nan_equal(got, want2.view(torch.int16).numpy().view(np.uint16), nan, 0x7FFF)
    assert ok, f"{bad} mismatches vs RNE(exact sum)"


def test_f32_add_matches_numpy():
    rng = np.random.default_rng(2)
    a = rng.integers(0, 1 << 32, 1 << 20, dtype=np.uint32).view(np.float32)
    b = rng.integers(0, 1 << 32, 1 << 20, dtype=np.uint32).view(np.float32)
    got = oracle.reduce("float32", "sum", a.copy(), b.copy())
    with np.errstate(all="ignore"):
        want = a + b
    nan = np.isnan(want)
    ok, bad = _canon_nan_equal(got.view(np.uint32), want.view(np.uint32), nan, 0x7FFFFFFF)
    assert ok, f"{bad} mismatches"


def test_f16_round_trip_all_halves_and_float_to_half_rounding():
    """The oracle's own half conversions: x + 0 must return every non-NaN half unchanged (exercises
    half->float->half on all 65536 patterns; -0 + +0 = +0 under RNE), and float sums that land
    between halves must round like numpy's astype(float16)."""
    allh = np.arange(1 << 16, dtype=np.uint16)
    zero = np.zeros_like(allh)
    got = oracle.reduce("float16", "sum", allh, zero)
    nan = np.isnan(allh.view(np.float16))
    want = allh.copy()
    want[allh == 0x8000] = 0x0000
    ok, bad = _canon_nan_equal(got, want, nan, 0x7FFF)
    assert ok, f"{bad} halves changed by x + 0"


@pytest.mark.parametrize("dtype", ["float32", "float16", "bfloat16", "int32"])
@pytest.mark.parametrize("redop", ["max", "min"])
def test_max_min_match_torch(dtype, redop):
    """Extension (the reference runtime only sums): torch.maximum / minimum semantics, NaN propagating."""
    g = torch.Generator().manual_seed(3)
    if dtype == "int32":
        a = torch.randint(-2**31, 2**31 - 1, (1 << 16,), generator=g, dtype=torch.int64).to(torch.int32)
        b = torch.randint(-2**31, 2**31 - 1, (1 << 16,), generator=g, dtype=torch.int64).to(torch.int32)
    else:
        a = (torch.randn(1 << 16, generator=g) * 4).to(TORCH_DTYPE[dtype])
        b = (torch.randn(1 << 16, generator=g) * 4).to(TORCH_DTYPE[dtype])
        a[:4] = torch.tensor([float("nan"), 1.0, float("inf"), float("-inf")]).to(a.dtype)
        b[:4] = torch.tensor([1.0, float("nan"), 1.0, 1.0]).to(a.dtype)
    got = from_raw(oracle.reduce(dtype, redop, to_raw(a), to_raw(b)), dtype)
    want = torch.maximum(a, b) if redop == "max" else torch.minimum(a, b)
    if dtype == "int32":
        assert torch.equal(got, want)
    else:
        nan = torch.isnan(want)
        assert torch.equal(torch.isnan(got), nan)
        assert torch.equal(got[~nan], want[~nan])


@pytest.mark.parametrize("dtype", ["float32", "float16", "bfloat16"])
def test_max_min_order_the_two_zeros(dtype):
    """IEEE 754-2019 maximum / minimum: -0 orders below +0 whatever the operand order (torch and numpy
    leave the sign of such a tie to the operand order, so this is pinned by its known answers), and
    equal operands come back unchanged."""
    neg = {"float32": 0x80000000, "float16": 0x8000, "bfloat16": 0x8000}[dtype]
    one = {"float32": 0x3F800000, "float16": 0x3C00, "bfloat16": 0x3F80}[dtype]
    raw = np.uint32 if dtype == "float32" else np.uint16
    a = np.array([0, neg, 0, neg, one, one | neg], dtype=raw)
    b = np.array([neg, 0, 0, neg, one, one | neg], dtype=raw)
    assert oracle.reduce(dtype, "max", a, b).tolist() == [0, 0, 0, neg, one, one | neg]
    assert oracle.reduce(dtype, "min", a, b).tolist() == [neg, neg, 0, neg, one, one | neg]


@pytest.mark.parametrize("dtype", ["float8_e4m3", "float8_e5m2"])
def test_fp8_sum_all_pairs_match_torch(dtype):
    """Reference vec.h:272-426: widen to f16, one f16 add, narrow with round-to-nearest-even and
    saturation to the largest finite value.  Independent authority: torch's CPU float8 <-> float16
    conversions and float16 add over all 65,536 operand pairs; the saturation is a clamp in f16
    before narrowing (every value between the largest finite one and its rounding boundary rounds
    down to it either way).  NaN results are compared as "is NaN" plus the oracle's documented
    canonical byte 0x7F."""
    td = TORCH_DTYPE[dtype]
    codes = torch.arange(256, dtype=torch.int16).to(torch.uint8)
    a = codes.repeat_interleave(256)
    b = codes.repeat(256)
    got = oracle.reduce(dtype, "sum", a.numpy().copy(), b.numpy().copy())
    s16 = a.view(td).to(torch.float16) + b.view(td).to(torch.float16)
    nan = torch.isnan(s16)
    want = s16.clamp(-FP8_MAX[dtype], FP8_MAX[dtype]).to(td).view(torch.uint8).numpy()
    assert nan.sum() > 0
    assert (got[nan.numpy()] == 0x7F).all()
    assert np.array_equal(got[~nan.numpy()], want[~nan.numpy()])
    # the widening itself: every code decodes to what torch decodes it to (x + (+0) keeps x, except
    # that -0 + +0 = +0)
    z = oracle.reduce(dtype, "sum", codes.numpy().copy(), np.zeros(256, np.uint8))
    fin = ~torch.isnan(codes.view(td).to(torch.float32)).numpy()
    back = torch.from_numpy(z).view(td).to(torch.float32).numpy()
    orig = codes.view(td).to(torch.float32).numpy()
    assert np.array_equal(back[fin], np.clip(orig[fin], -FP8_MAX[dtype], FP8_MAX[dtype]))


@pytest.mark.parametrize("dtype", ["float8_e4m3", "float8_e5m2"])
@pytest.mark.parametrize("redop", ["max", "min"])
def test_fp8_max_min_all_pairs(dtype, redop):
    """Extension: NaN-propagating selection; infinities (e5m2) saturate on the way out like every
    other result of the fp8 path."""
    td = TORCH_DTYPE[dtype]
    codes = torch.arange(256, dtype=torch.int16).to(torch.uint8)
    a = codes.repeat_interleave(256)
    b = codes.repeat(256)
    got = oracle.reduce(dtype, redop, a.numpy().copy(), b.numpy().copy())
    fa, fb = a.view(td).to(torch.float32), b.view(td).to(torch.float32)
    sel = torch.maximum(fa, fb) if redop == "max" else torch.minimum(fa, fb)
    nan = torch.isnan(sel).numpy()
    assert (got[nan] == 0x7F).all()
    back = torch.from_numpy(got).view(td).to(torch.float32).numpy()
    assert np.array_equal(back[~nan], np.clip(sel.numpy()[~nan], -FP8_MAX[dtype], FP8_MAX[dtype]))


def test_int32_sum_wraps():
    a = np.array([2**31 - 1, -2**31, 5, -7], dtype=np.int32)
    b = np.array([1, -1, -9, 7], dtype=np.int32)
    got = oracle.reduce("int32", "sum", a, b)
    assert got.tolist() == [-2**31, 2**31 - 1, -4, 0]


# ------------------------------------------------------------------------------- closed forms

def _run(alg, method, world, n, dtype, inputs, channels=1, executor="tma", place=None, buffer_elems=0, **ext):
    jsons = graph_jsons(alg, method, world, n, dtype, executor, channels, **ext)
    return oracle_buffers(jsons, inputs, dtype, place=place, buffer_elems=buffer_elems), jsons


@pytest.mark.parametrize("world", [2, 4, 8])
def test_allreduce_rank_plus_one_closed_form(world):
    """reference tests/test_correctness.py:142,170-171: input rank+1 -> R(R+1)/2, exact in bf16."""
    n = 1024 * world
    out, _ = _run("ring", "build_allreduce", world, n, "bfloat16", seeded_inputs("rank+1", world, n, "bfloat16"))
    for r in range(world):
        assert torch.all(out[r].float() == world * (world + 1) / 2)


@pytest.mark.parametrize("alg", ["rhd", "tree"])
def test_log_step_allreduce_closed_form(alg):
    world, n = 8, 4096
    out, _ = _run(alg, "build_allreduce", world, n, "bfloat16", seeded_inputs("rank+1", world, n, "bfloat16"))
    for r in range(world):
        assert torch.all(out[r].float() == 36.0)


def test_reduce_scatter_closed_form():
    """reference tests/test_correctness.py:196-217: chunk r of rank r holds the full sum."""
    world, n = 4, 4096
    chunk = n // world
    out, _ = _run("ring", "build_reduce_scatter", world, n, "bfloat16", seeded_inputs("rank+1", world, n, "bfloat16"))
    for r in range(world):
        assert torch.all(out[r][r * chunk:(r + 1) * chunk].float() == 10.0)


def test_allgather_closed_form():
    """reference tests/test_correctness.py:219-241: input chunk staged at rank*chunk; every rank ends
    with chunk i = i+1."""
    world, n = 4, 4096
    chunk = n // world
    parts = [torch.full((chunk,), r + 1, dtype=torch.bfloat16) for r in range(world)]
    out, _ = _run("ring", "build_allgather", world, n, "bfloat16", parts, place=lambda r: r * chunk, buffer_elems=n)
    for r in range(world):
        for i in range(world):
            assert torch.all(out[r][i * chunk:(i + 1) * chunk].float() == i + 1)


def test_alltoall_closed_form():
    """reference tests/test_correctness.py:243-272 with the engine's assembly rule
    (csrc/engine_c.cc:524-543): own chunk from the data region, partner p's from scratch."""
    world, n = 4, 4096
    chunk = n // world
    inputs = [torch.cat([torch.full((chunk,), r * 100 + i, dtype=torch.bfloat16) for i in range(world)])
              for r in range(world)]
    out, _ = _run("ring", "build_alltoall", world, n, "bfloat16", inputs, buffer_elems=2 * n)
    for r in range(world):
        for p in range(world):
            src = r * chunk if p == r else n + p * chunk
            want = torch.tensor(float(p * 100 + r)).to(torch.bfloat16)   # 301 etc. round in bf16
            assert torch.all(out[r][src:src + chunk] == want)


# ------------------------------------------------------------------------------- reduction order

def _fl(x, dtype):
    return x.to(TORCH_DTYPE[dtype])


def ring_order(x, world, channels, dtype):
    """chunk c: acc = x_c; for k = 1..R-1: acc = fl(x_{(c+k) mod R} + acc) — from the schedule:
    rank r at step s reduces chunk (r-s-1) pulled from rank r-1."""
    n = x[0].numel()
    per_ch = n // channels
    per_rank = per_ch // world
    out = torch.empty_like(x[0])
    for ch in range(channels):
        for c in range(world):
            lo = ch * per_ch + c * per_rank
            acc = x[c][lo:lo + per_rank].clone()
            for k in range(1, world):
                acc = x[(c + k) % world][lo:lo + per_rank] + acc
            out[lo:lo + per_rank] = acc
    return out


def rhd_order(x, world, dtype):
    """v_r^(k+1) = fl(v_{r xor 2^k}^(k) + v_r^(k)) on the half rank r keeps: a pairwise tree by rank
    bits, low bit first.  Evaluated per position: which ranks contribute in which grouping depends
    only on the rank bits, so the whole tensor follows one formula."""
    v = [t.clone() for t in x]
    k = 1
    while k < world:
        v = [v[r ^ k] + v[r] for r in range(world)]   # IEEE add commutes: both partners get the same bits
        k <<= 1
    return v[0]


def tree_order(x, world, dtype):
    """level k: every rank with low k+1 bits zero does v_r = fl(v_{r+2^k} + v_r)."""
    v = [t.clone() for t in x]
    k = 1
    while k < world:
        for r in range(0, world, 2 * k):
            v[r] = v[r + k] + v[r]
        k <<= 1
    return v[0]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16", "float16"])
@pytest.mark.parametrize("alg,world,channels", [("ring", 8, 1), ("ring", 4, 2), ("ring", 3, 1),
                                                ("rhd", 8, 1), ("rhd", 16, 1), ("tree", 8, 1), ("tree", 32, 1)])
def test_reduction_order_brute_force(alg, world, channels, dtype):
    n = 64 * world * channels
    kind = "randn0.1" if dtype == "float16" else "randn"
    x = seeded_inputs(kind, world, n, dtype, seed=11)
    out, _ = _run(alg, "build_allreduce", world, n, dtype, x, channels=channels, executor="sm")
    if alg == "ring":
        want = ring_order(x, world, channels, dtype)
    elif alg == "rhd":
        want = rhd_order(x, world, dtype)
    else:
        want = tree_order(x, world, dtype)
    for r in range(world):
        assert bits_equal(out[r], want), f"rank {r}: {mismatch_report(out[r], want)}"
    # tolerance clause: close to the float64 sum
    exact = sum(t.double() for t in x)
    tol = {"float32": 1e-6 * world, "bfloat16": 1e-2 * world, "float16": 2e-3 * world}[dtype]
    assert torch.all((out[0].double() - exact).abs() <= tol * exact.abs().clamp_min(1.0))


def test_order_insensitive_results_match_stack_reductions():
    """int32 SUM (wraps) and MAX: any order gives the same bits as torch over the stacked inputs."""
    world, n = 8, 1024
    xi = seeded_inputs("randint", world, n, "int32", seed=2)
    xi[0][:8] = 2**31 - 5    # force wraparound
    out, _ = _run("tree", "build_allreduce", world, n, "int32", xi, executor="sm")
    want = torch.stack(xi).to(torch.int64).sum(0).to(torch.int32)    # int64 sum truncated = mod 2^32
    assert torch.equal(out[3], want)
    xf = seeded_inputs("randn", world, n, "float32", seed=4)
    out, _ = _run("tree", "build_allreduce", world, n, "float32", xf, executor="sm", reduce_op="max")
    assert torch.equal(out[5], torch.stack(xf).amax(0))


# ------------------------------------------------------------------------------- runner semantics

@pytest.mark.parametrize("alg,world,channels", [("ring", 8, 4), ("rhd", 8, 2), ("tree", 8, 1)])
def test_result_does_not_depend_on_the_interleaving(alg, world, channels):
    n = 128 * world * channels
    x = seeded_inputs("randn", world, n, "float32", seed=7)
    jsons = graph_jsons(alg, "build_allreduce", world, n, "float32", "sm", channels)
    base = oracle_buffers(jsons, x, "float32", sched_seed=0)
    for seed in (1, 2, 12345):
        other = oracle_buffers(jsons, x, "float32", sched_seed=seed)
        for r in range(world):
            assert bits_equal(base[r], other[r])


def test_algorithmic_byte_closed_forms():
    """ring 5(R-1)S, ring RS 3(R-1)S, ring AG 2(R-1)S, RHD 5(1-1/R)RS, tree 5(R-1)S; balanced signals."""
    world, n = 8, 8192
    S = n * 4
    cases = {("ring", "build_allreduce"): 5 * (world - 1) * S, ("ring", "build_reduce_scatter"): 3 * (world - 1) * S,
             ("ring", "build_allgather"): 2 * (world - 1) * S, ("rhd", "build_allreduce"): 5 * (world - 1) * S,
             ("tree", "build_allreduce"): 5 * (world - 1) * S}
    for (alg, method), want in cases.items():
        graphs = [oracle.Graph(json.loads(j)) for j in graph_jsons(alg, method, world, n, "float32")]
        bufs = [np.zeros(n, dtype=np.float32) for _ in range(world)]
        st = oracle.run(graphs, bufs)
        assert st.bytes == want, (alg, method)
        assert st.residual == 0 and st.deadlocked == 0


def test_wait_without_notify_is_reported_as_deadlock():
    from pccl_amd.dsl import CommunicationOp, compile_to_json_string
    jsons = []
    for rank in range(2):
        with CommunicationOp(name=f"dl{rank}") as op:
            op.tensor(dtype="float32", shape=(16,))
            op.wait_notify(signal_id=7, source_rank=1 - rank)    # nobody ever notifies 7
            op.sm_copy(source_rank=1 - rank, src_offset=0, dst_offset=0, size=16)
        jsons.append(compile_to_json_string(op.get_graph()))
    graphs = [oracle.Graph(json.loads(j)) for j in jsons]
    with pytest.raises(oracle.OracleError, match="deadlock"):
        oracle.run(graphs, [np.zeros(16, dtype=np.float32) for _ in range(2)])


def test_counts_carried_from_one_execution_to_the_next():
    """The reference keeps one signal region per engine and clears it only in Engine::resetSignals
    (csrc/engine_c.cc:131-146, 576-593); a wait passes on a count above zero and takes one
    (cuda_executor.cu:425-445).  Known answers that follow from those two functions alone: an
    operation whose only wait has no notify deadlocks from zero and runs, once per count, on what
    earlier executions left; k executions of an operation with n notifies and w waits on a semaphore
    move it by k (n - w); clearing the region brings the deadlock back.  Buffers against numpy."""
    n = 64
    ops = {k: [oracle.Graph(json.loads(j)) for j in v] for k, v in carry_ops(n).items()}
    rng = np.random.default_rng(5)
    bufs = [rng.standard_normal(n).astype(np.float32) for _ in range(2)]
    sig = oracle.new_signals(2)

    def state():
        return {(int(r), int(i)): int(sig[r, i]) for r, i in zip(*np.nonzero(sig))}

    def step(name):
        nonlocal bufs
        want = carry_expected(name, bufs)
        oracle.run(ops[name], bufs, signals=sig)
        for got, w in zip(bufs, want):
            assert np.array_equal(got.view(np.int32), w.view(np.int32)), name
    with pytest.raises(oracle.OracleError, match="deadlock"):
        oracle.run(ops["take"], [b.copy() for b in bufs], signals=oracle.new_signals(2))
    step("give"); assert state() == {(1, 5): 1}
    step("take"); assert state() == {}
    with pytest.raises(oracle.OracleError, match="deadlock"):
        oracle.run(ops["take"], [b.copy() for b in bufs], signals=sig.copy())
    for k in range(1, 4):
        step("give"); assert state() == {(1, 5): k}
    step("pair"); assert state() == {(1, 5): 3}          # balanced: leaves what it found
    for k in (2, 1, 0):
        step("take"); assert state() == ({(1, 5): k} if k else {})
    # without a state handed in every execution starts from zero, as before
    oracle.run(ops["give"], bufs)
    with pytest.raises(oracle.OracleError, match="deadlock"):
        oracle.run(ops["take"], bufs)
    # resetSignals: the region is zeroed, the deadlock is back
    step("give"); sig[:] = 0
    with pytest.raises(oracle.OracleError, match="deadlock"):
        oracle.run(ops["take"], bufs, signals=sig)


def test_out_of_range_access_is_an_error():
    jsons = graph_jsons("ring", "build_allreduce", 2, 2048, "float32", "sm")
    graphs = [oracle.Graph(json.loads(j)) for j in jsons]
    with pytest.raises(oracle.OracleError, match="outside"):
        oracle.run(graphs, [np.zeros(1024, dtype=np.float32) for _ in range(2)])


def test_ragged_sub_ops_process_every_element():
    """Extension: sub-op boundaries off 16-byte alignment (the reference would drop tails)."""
    from pccl_amd.dsl import ragged_cuts
    world, n = 4, 4099
    cuts = ragged_cuts(n, 6, seed=1)
    assert all(c % 4 for c in cuts)
    x = seeded_inputs("randint", world, n, "int32", seed=8)
    out, _ = _run("tree", "build_allreduce", world, n, "int32", x, executor="sm", cuts=cuts)
    want = torch.stack(x).sum(0).to(torch.int32)
    for r in range(world):
        assert torch.equal(out[r], want)
