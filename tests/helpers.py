"""Shared test utilities: graph generation, seeded inputs, and the oracle leg.

The oracle (oracle/) is imported here and only here on the test side; the product package never
sees it.
"""
from __future__ import annotations

import json
import os
import sys
from typing import List, Sequence

import numpy as np
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

from oracle import oracle  # noqa: E402
from pccl_amd.dsl import ALGORITHMS, CommunicationOp, Pipeline, compile_to_json_string  # noqa: E402

GOLDEN = os.path.join(ROOT, "tests", "golden")

TORCH_DTYPE = {"float32": torch.float32, "float16": torch.float16, "bfloat16": torch.bfloat16,
               "int32": torch.int32, "float8_e4m3": torch.float8_e4m3fn, "float8_e5m2": torch.float8_e5m2}
RAW_NP = {"float32": np.float32, "float16": np.uint16, "bfloat16": np.uint16, "int32": np.int32,
          "float8_e4m3": np.uint8, "float8_e5m2": np.uint8}
FP8_MAX = {"float8_e4m3": 448.0, "float8_e5m2": 57344.0}


def graph_jsons(alg: str, method: str, world: int, n: int, dtype: str, executor: str = "sm",
                channels: int = 1, **ext) -> List[str]:
    a = ALGORITHMS[alg]()
    return [compile_to_json_string(getattr(a, method)(r, world, n, dtype=dtype, executor=executor,
                                                      num_channels=channels, **ext))
            for r in range(world)]


def pipelined_ring_allreduce(rank: int, world: int, n: int, dtype: str, depth: int, reduce_op: str = "sum",
                             paired_signals: bool = False):
    """Ring allreduce whose steps rotate over `depth` channels through the Pipeline construct.

    paired_signals=False numbers the signals exactly as the reference's bandwidth script does
    (tests/bench_allreduce_tma_bw.py:119-186: one running counter over waits and notifies).  That
    numbering makes step s+1 wait on an id nobody notifies.  The reference's wait spins until the
    count is above zero and has no bail-out (cuda_executor.cu:946-961; only the other blocks'
    channel barrier at :997-1003 gives up, after 4 M spins), so there the schedule can only finish
    on counts that earlier executions left in the signal array, which is never cleared between
    executions (engine_c.cc:576-593); exact semaphore semantics from zero report a deadlock.
    paired_signals=True is the same schedule with the wait of step t+1 on the id step t
    of the previous rank notifies, which is executable."""
    chunk = n // world
    prev_rank, next_rank = (rank - 1) % world, (rank + 1) % world
    steps = [("reduce", ((rank - s - 1) % world) * chunk) for s in range(world - 1)] + \
            [("copy", ((rank - s) % world) * chunk) for s in range(world - 1)]
    with CommunicationOp(name=f"ar_pipe{depth}_rank{rank}") as op:
        op.tensor(dtype=dtype, shape=(n,))
        pipe = Pipeline(depth=depth)
        sig = 0
        with pipe.bind(op):
            for _ in range(depth):
                with pipe.stage():
                    sig += 1
                    op.notify(signal_id=sig, target_rank=next_rank)
                    op.wait_notify(signal_id=sig, source_rank=prev_rank)
            for t, (kind, off) in enumerate(steps):
                with pipe.stage():
                    if paired_signals:
                        if t > 0:
                            op.wait_notify(signal_id=100 + t - 1, source_rank=prev_rank)
                    elif t > 0:
                        sig += 1
                        op.wait_notify(signal_id=sig, source_rank=prev_rank)
                    if kind == "reduce":
                        op.sm_reduce(reduce_op=reduce_op, source_rank=prev_rank, src_offset=off, dst_offset=off,
                                     remote_offset=off, count=chunk)
                    else:
                        op.sm_copy(source_rank=prev_rank, src_offset=off, dst_offset=off, size=chunk)
                    sig += 1
                    op.notify(signal_id=100 + t if paired_signals else sig, target_rank=next_rank)
            if paired_signals:
                with pipe.stage():
                    op.wait_notify(signal_id=100 + len(steps) - 1, source_rank=prev_rank)
            else:
                for _ in range(depth):
                    with pipe.stage():
                        sig += 1
                        op.wait_notify(signal_id=sig, source_rank=prev_rank)
        return op.get_graph()


def chained_gather(rank: int, world: int, chunk: int, dtype: str, pieces: int, kind: str):
    """`pieces` same-type data ops from the next rank whose source ranges follow one another, a
    notify / wait pair after every second one, closed by a notify / wait: the shape of chain the
    channelize pass (reference pccl/dsl/passes/channelize.py) looks for."""
    peer = (rank + 1) % world
    with CommunicationOp(name=f"chain_{kind}_rank{rank}") as op:
        op.tensor(dtype=dtype, shape=(pieces * chunk,))
        op.notify(signal_id=1, target_rank=(rank - 1) % world)
        op.wait_notify(signal_id=1, source_rank=peer)
        for k in range(pieces):
            if kind == "copy":
                op.sm_copy(source_rank=peer, src_offset=k * chunk, dst_offset=k * chunk, size=chunk)
            else:
                op.tma_reduce(reduce_op="sum", source_rank=peer, src_offset=k * chunk, dst_offset=k * chunk,
                              remote_offset=k * chunk, count=chunk)
            if k % 2 == 1:
                op.notify(signal_id=10 + k, target_rank=(rank - 1) % world)
                op.wait_notify(signal_id=10 + k, source_rank=peer)
        op.notify(signal_id=2, target_rank=(rank - 1) % world)
        op.wait_notify(signal_id=2, source_rank=peer)
        return op.get_graph()


def random_program(seed: int, world: int, n: int, num_ops: int, dtype: str, aligned: bool,
                   reduce_ops=("sum",)) -> List[str]:
    """A random race-free program: `num_ops` reduces and copies over random ranks, peers and element
    ranges (sizes and offsets of any parity), in one global order that notify / wait pairs enforce
    from each op to the next (program order where both are on one rank).  With aligned=True every
    op reads and writes the same element positions (the column runner's domain); otherwise source
    and destination ranges differ (reduce: the own operand is read where the result is written).
    Returns the per-rank JSON graphs."""
    rng = np.random.default_rng(seed)
    builders = []
    for r in range(world):
        op = CommunicationOp(name=f"rand{seed}_rank{r}")
        op.__enter__()
        op.tensor(dtype=dtype, shape=(n,))
        builders.append(op)
    prev_rank, used = None, [False] * world
    for k in range(num_ops):
        r = int(rng.integers(world))
        peer = int(rng.integers(world - 1))
        peer += peer >= r
        size = int(rng.integers(1, max(2, n // 3)))
        dst = int(rng.integers(0, n - size + 1))
        src = dst if aligned else int(rng.integers(0, n - size + 1))
        if prev_rank is not None and prev_rank != r:
            builders[prev_rank].notify(signal_id=k, target_rank=r)
            builders[r].wait_notify(signal_id=k, source_rank=prev_rank)
        if rng.random() < 0.5:
            builders[r].sm_reduce(reduce_op=str(rng.choice(reduce_ops)), source_rank=peer, remote_offset=src,
                                  src_offset=dst, dst_offset=dst, count=size)
        else:
            builders[r].sm_copy(source_rank=peer, src_offset=src, dst_offset=dst, size=size)
        prev_rank, used[r] = r, True
    out = []
    for r, op in enumerate(builders):
        if not used[r]:          # a rank with nothing to do still registers a graph
            op.sm_copy(source_rank=(r + 1) % world, src_offset=0, dst_offset=0, size=0)
        op.__exit__(None, None, None)
        out.append(compile_to_json_string(op.get_graph()))
    return out


def carry_ops(n: int = 64, dtype: str = "float32") -> dict:
    """Two-rank operations whose notifies and waits do not balance, for the semaphore state that the
    reference keeps from one execution to the next (csrc/engine_c.cc:576-593).  h = n / 2.
      give  rank 0: own[0:h] <- rank 1's [0:h]; notify (1, 5) twice.   rank 1: wait 5; own[h:n] <- rank 0's [h:n].
            One notify is left over: (1, 5) goes up by one.
      take  rank 0: own[h:n] <- rank 1's [h:n].   rank 1: wait 5 (nobody notifies it here); own[0:h] += rank 0's [0:h].
            Runs only on a count that an earlier execution left: (1, 5) goes down by one.
      pair  rank 0: own[0:h] += rank 1's [0:h]; notify (1, 5).   rank 1: wait 5; own[h:n] <- rank 0's [0:h].
            Balanced, and race-free from zero; on a carried count the wait passes before the notify and
            rank 1's copy is no longer ordered after rank 0's reduce: a data race."""
    h = n // 2

    def build(rank, body):
        with CommunicationOp(name=f"carry{rank}") as op:
            op.tensor(dtype=dtype, shape=(n,))
            body(op)
        return compile_to_json_string(op.get_graph())

    return {
        "give": [build(0, lambda op: (op.sm_copy(source_rank=1, src_offset=0, dst_offset=0, size=h),
                                      op.notify(signal_id=5, target_rank=1), op.notify(signal_id=5, target_rank=1))),
                 build(1, lambda op: (op.wait_notify(signal_id=5, source_rank=0),
                                      op.sm_copy(source_rank=0, src_offset=h, dst_offset=h, size=n - h)))],
        "take": [build(0, lambda op: op.sm_copy(source_rank=1, src_offset=h, dst_offset=h, size=n - h)),
                 build(1, lambda op: (op.wait_notify(signal_id=5, source_rank=0),
                                      op.sm_reduce(source_rank=0, remote_offset=0, src_offset=0, dst_offset=0, count=h)))],
        "pair": [build(0, lambda op: (op.sm_reduce(source_rank=1, remote_offset=0, src_offset=0, dst_offset=0, count=h),
                                      op.notify(signal_id=5, target_rank=1))),
                 build(1, lambda op: (op.wait_notify(signal_id=5, source_rank=0),
                                      op.sm_copy(source_rank=0, src_offset=0, dst_offset=h, size=h)))],
    }


def carry_expected(name: str, bufs: Sequence[np.ndarray]) -> List[np.ndarray]:
    """What one execution of a ``carry_ops`` operation leaves in the two rank buffers, written from the
    operation's description with numpy (float32 or int32 arrays)."""
    a, b = bufs[0].copy(), bufs[1].copy()
    h = len(a) // 2
    if name == "give":
        a[:h], b[h:] = bufs[1][:h], bufs[0][h:]
    elif name == "take":
        a[h:], b[:h] = bufs[1][h:], bufs[0][:h] + bufs[1][:h]
    elif name == "pair":
        a[:h] = bufs[1][:h] + bufs[0][:h]
        b[h:2 * h] = a[:h]
    else:
        raise KeyError(name)
    return [a, b]


def to_raw(t: torch.Tensor) -> np.ndarray:
    """CPU tensor -> numpy array of its storage bits (bf16/f16 as uint16)."""
    t = t.contiguous()
    if t.dtype in (torch.bfloat16, torch.float16):
        return t.view(torch.int16).numpy().view(np.uint16).copy()
    if t.dtype in (torch.float8_e4m3fn, torch.float8_e5m2):
        return t.view(torch.uint8).numpy().copy()
    return t.numpy().copy()


def from_raw(a: np.ndarray, dtype: str) -> torch.Tensor:
    if dtype in ("bfloat16", "float16"):
        return torch.from_numpy(a.view(np.int16).copy()).view(TORCH_DTYPE[dtype])
    if dtype in FP8_MAX:
        return torch.from_numpy(a.view(np.uint8).copy()).view(TORCH_DTYPE[dtype])
    return torch.from_numpy(a.copy())


def seeded_inputs(kind: str, world: int, n: int, dtype: str, seed: int = 0) -> List[torch.Tensor]:
    """CPU-generator inputs, one row per rank, as the configurations prescribe."""
    g = torch.Generator().manual_seed(seed)
    if kind == "randn":
        x = torch.randn(world, n, generator=g)
    elif kind == "uniform":
        x = torch.rand(world, n, generator=g) * 2 - 1
    elif kind == "randn0.1":
        x = torch.randn(world, n, generator=g) * 0.1
    elif kind == "randint":
        x = torch.randint(-1000, 1000, (world, n), generator=g)
    elif kind == "rank+1":
        x = torch.arange(1, world + 1).view(world, 1).expand(world, n).float()
    else:
        raise ValueError(kind)
    if dtype in FP8_MAX:   # torch's conversion does not saturate; keep the draw inside the finite range
        x = x.clamp(-FP8_MAX[dtype], FP8_MAX[dtype])
    return [x[r].to(TORCH_DTYPE[dtype]).contiguous() for r in range(world)]


def oracle_buffers(jsons: Sequence[str], inputs: Sequence[torch.Tensor], dtype: str,
                   sched_seed: int = 0, buffer_elems: int = 0, place=None,
                   threads: int = 0) -> List[torch.Tensor]:
    """Run the graphs on the CPU oracle.  Rank r's buffer starts as zeros with inputs[r] copied in
    at element offset place(r) (default 0); returns the final buffers."""
    graphs = [oracle.Graph(json.loads(j)) for j in jsons]
    n = max(buffer_elems, max(len(x) + (place(r) if place else 0) for r, x in enumerate(inputs)))
    bufs = []
    for r, x in enumerate(inputs):
        raw = np.zeros(n, dtype=RAW_NP[dtype])
        off = place(r) if place else 0
        raw[off:off + len(x)] = to_raw(x)
        bufs.append(raw)
    oracle.run(graphs, bufs, sched_seed=sched_seed, threads=threads)
    return [from_raw(b, dtype) for b in bufs]


def bits_equal(a: torch.Tensor, b: torch.Tensor) -> bool:
    a, b = a.cpu().contiguous(), b.cpu().contiguous()
    if a.dtype in (torch.bfloat16, torch.float16):
        return torch.equal(a.view(torch.int16), b.view(torch.int16))
    if a.dtype == torch.float32:
        return torch.equal(a.view(torch.int32), b.view(torch.int32))
    if a.dtype in (torch.float8_e4m3fn, torch.float8_e5m2):
        return torch.equal(a.view(torch.uint8), b.view(torch.uint8))
    return torch.equal(a, b)


def mismatch_report(a: torch.Tensor, b: torch.Tensor) -> str:
    a, b = a.cpu(), b.cpu()
    if a.dtype in (torch.bfloat16, torch.float16):
        ne = (a.view(torch.int16) != b.view(torch.int16)).nonzero().flatten()
    elif a.dtype == torch.float32:
        ne = (a.view(torch.int32) != b.view(torch.int32)).nonzero().flatten()
    elif a.dtype in (torch.float8_e4m3fn, torch.float8_e5m2):
        a, b = a.view(torch.uint8), b.view(torch.uint8)
        ne = (a != b).nonzero().flatten()
    else:
        ne = (a != b).nonzero().flatten()
    if len(ne) == 0:
        return "equal"
    i = int(ne[0])
    return f"{len(ne)} of {a.numel()} differ; first at {i}: got {a[i].item()} expected {b[i].item()}"
