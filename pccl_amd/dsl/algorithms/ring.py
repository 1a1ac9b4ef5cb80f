"""Ring schedules: allreduce, reduce-scatter, allgather, alltoall.

Same schedule, offsets and signal ids as reference pccl/dsl/algorithms/ring.py:
per channel ``c`` the slice ``[c*N/C, (c+1)*N/C)`` is cut into ``R`` chunks; signal ``c*1000+100``
is the start barrier and ``c*1000`` the per-step "chunk ready" semaphore; every data op pulls
from ``prev = rank-1`` and is followed by a notify to ``next = rank+1``.
"""
from __future__ import annotations

from ..builder import CommunicationOp, Stream
from ..ir import Graph
from .base import CollectiveAlgorithm, _Emit


def _ring_phase_graph(kind: str, first_chunk_shift, phases, rank, world_size, tensor_size,
                      dtype, executor, num_channels, reduce_op, cuts, collective) -> Graph:
    """Shared skeleton.  ``phases`` is a list of ("reduce"|"copy", chunk_shift) pairs: phase p,
    step s touches chunk ``(rank - s - shift) mod R``.  The very first data op of a channel is
    gated by the start barrier only; every later one waits on the step semaphore."""
    per_ch = tensor_size // num_channels
    per_rank = per_ch // world_size
    prev_rank, next_rank = (rank - 1) % world_size, (rank + 1) % world_size
    with CommunicationOp(name=f"ring_{kind}_{executor}_c{num_channels}_rank{rank}") as op:
        op.tensor(dtype=dtype, shape=(tensor_size,))
        em = _Emit(op, executor, reduce_op, cuts)
        for c in range(num_channels):
            base, sig = c * per_ch, c * 1000
            with Stream(f"ch{c}"):
                op.set_channel(c)
                op.notify(signal_id=sig + 100, target_rank=next_rank)
                op.wait_notify(signal_id=sig + 100, source_rank=prev_rank)
                first = True
                for what, shift in phases:
                    for step in range(world_size - 1):
                        off = base + ((rank - step - shift) % world_size) * per_rank
                        if not first:
                            op.wait_notify(signal_id=sig, source_rank=prev_rank)
                        first = False
                        (em.reduce if what == "reduce" else em.copy)(prev_rank, off, per_rank)
                        op.notify(signal_id=sig, target_rank=next_rank)
                op.wait_notify(signal_id=sig, source_rank=prev_rank)
    g = op.get_graph()
    g.collective_type = collective
    return g


class RingAllreduce(CollectiveAlgorithm):
    name = "ring"
    step_count = "O(2(N-1))"
    bandwidth_optimal = True

    def build_allreduce(self, rank, world_size, tensor_size, dtype="bfloat16", executor="tma",
                        num_channels=1, reduce_op="sum", cuts=None) -> Graph:
        # reduce-scatter on chunk (rank-s-1), then allgather on chunk (rank-s)
        return _ring_phase_graph("ar", None, [("reduce", 1), ("copy", 0)], rank, world_size,
                                 tensor_size, dtype, executor, num_channels, reduce_op, cuts,
                                 "allreduce")

    def build_reduce_scatter(self, rank, world_size, tensor_size, dtype="bfloat16",
                             executor="tma", num_channels=1, reduce_op="sum", cuts=None) -> Graph:
        # shift 2 so that the fully reduced chunk ends at position `rank`
        return _ring_phase_graph("rs", None, [("reduce", 2)], rank, world_size, tensor_size,
                                 dtype, executor, num_channels, reduce_op, cuts,
                                 "reduce_scatter")

    def build_allgather(self, rank, world_size, tensor_size, dtype="bfloat16", executor="tma",
                        num_channels=1, reduce_op="sum", cuts=None) -> Graph:
        # step 0 pulls prev's own chunk (position rank-1)
        return _ring_phase_graph("ag", None, [("copy", 1)], rank, world_size, tensor_size,
                                 dtype, executor, num_channels, reduce_op, cuts, "allgather")

    def build_alltoall(self, rank, world_size, tensor_size, dtype="bfloat16", executor="tma",
                       num_channels=1, **_ext) -> Graph:
        """N-1 barrier rounds, then direct pulls of chunk[rank] from every partner into the
        scratch region ``[tensor_size, 2*tensor_size)``; always SM copies
        (reference ring.py:195-246)."""
        per_ch = tensor_size // num_channels
        per_rank = per_ch // world_size
        prev_rank, next_rank = (rank - 1) % world_size, (rank + 1) % world_size
        with CommunicationOp(name=f"ring_a2a_sm_c{num_channels}_rank{rank}") as op:
            op.tensor(dtype=dtype, shape=(tensor_size,))
            for c in range(num_channels):
                base, sig = c * per_ch, c * 1000
                with Stream(f"ch{c}"):
                    op.set_channel(c)
                    for i in range(world_size - 1):
                        op.notify(signal_id=sig + 100 + i, target_rank=next_rank)
                        op.wait_notify(signal_id=sig + 100 + i, source_rank=prev_rank)
                    for step in range(world_size - 1):
                        partner = (rank + step + 1) % world_size
                        op.sm_copy(source_rank=partner, src_offset=base + rank * per_rank,
                                   dst_offset=base + tensor_size + partner * per_rank,
                                   size=per_rank)
        g = op.get_graph()
        g.collective_type = "alltoall"
        return g
