"""Recursive halving-doubling allreduce (reference pccl/dsl/algorithms/recursive_hd.py:32-145).

Step k pairs rank with ``rank ^ 2^k``.  Halving: the active region is split in two and the half
selected by bit k of the rank is reduced from the partner.  Doubling mirrors it in reverse with
copies.  Signal id = the sender's rank, so each (target, sender) pair owns one semaphore; every
step opens with a "my earlier ops are done" notify, and only the last doubling step is
acknowledged so all semaphores return to zero.

Extension: ``num_channels > 1`` (the reference always emits channel 0).  Channel ``c`` runs the
whole schedule on its own slice ``[c*N/C, (c+1)*N/C)`` of the tensor (halving that slice step by
step), on stream ``ch{c}`` with signal ids ``c*1000 + sender`` (the ring templates' id
convention), so channels never touch each other's positions.
"""
from __future__ import annotations

from ..builder import CommunicationOp, Stream
from ..ir import Graph
from .base import CollectiveAlgorithm, _Emit, require_power_of_two


class RecursiveHalvingDoubling(CollectiveAlgorithm):
    name = "rhd"
    step_count = "O(2 log N)"
    bandwidth_optimal = True

    def build_allreduce(self, rank, world_size, tensor_size, dtype="bfloat16", executor="tma",
                        num_channels=1, reduce_op="sum", cuts=None) -> Graph:
        log_n = require_power_of_two("RecursiveHalvingDoubling", world_size)

        per_ch = tensor_size // num_channels

        def region_start(k: int) -> int:
            return sum(per_ch >> (j + 1) for j in range(k) if rank >> j & 1)

        with CommunicationOp(name=f"rhd_ar_{executor}_rank{rank}") as op:
            op.tensor(dtype=dtype, shape=(tensor_size,))
            em = _Emit(op, executor, reduce_op, cuts)
            for c in range(num_channels):
                sig, base = c * 1000, c * per_ch
                with Stream("main" if num_channels == 1 else f"ch{c}"):
                    op.set_channel(c)
                    for k in range(log_n):
                        partner, seg = rank ^ (1 << k), per_ch >> (k + 1)
                        keep = base + region_start(k) + (seg if rank >> k & 1 else 0)
                        op.notify(signal_id=sig + rank, target_rank=partner)
                        op.wait_notify(signal_id=sig + partner, source_rank=partner)
                        em.reduce(partner, keep, seg)
                    for k in range(log_n - 1, -1, -1):
                        partner, seg = rank ^ (1 << k), per_ch >> (k + 1)
                        fetch = base + region_start(k) + (0 if rank >> k & 1 else seg)
                        op.notify(signal_id=sig + rank, target_rank=partner)
                        op.wait_notify(signal_id=sig + partner, source_rank=partner)
                        em.copy(partner, fetch, seg)
                        if k == 0:
                            op.notify(signal_id=sig + rank, target_rank=partner)
                    op.wait_notify(signal_id=sig + (rank ^ 1), source_rank=rank ^ 1)
        g = op.get_graph()
        g.collective_type = "allreduce"
        return g
