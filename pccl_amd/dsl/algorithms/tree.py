"""Binary-tree allreduce (reference pccl/dsl/algorithms/tree.py:30-123).

Reduce phase: at level k every rank whose low k+1 bits are zero pulls the whole tensor from
``rank + 2^k`` and adds it; a rank drops out after it has been pulled from.  Broadcast phase
walks the levels back down with copies.  Signal id = the sender's rank.

Extensions: ``num_channels > 1`` (slice ``[c*N/C, (c+1)*N/C)`` on stream ``ch{c}``, ids
``c*1000 + sender``), ``reduce_op`` and ragged ``cuts`` (each whole-tensor op becomes a run of
consecutive sub-ops between the same wait/notify pair).
"""
from __future__ import annotations

from ..builder import CommunicationOp, Stream
from ..ir import Graph
from .base import CollectiveAlgorithm, _Emit, require_power_of_two


class TreeAllreduce(CollectiveAlgorithm):
    name = "tree"
    step_count = "O(2 log N)"
    bandwidth_optimal = False

    def build_allreduce(self, rank, world_size, tensor_size, dtype="bfloat16", executor="tma",
                        num_channels=1, reduce_op="sum", cuts=None) -> Graph:
        log_n = require_power_of_two("TreeAllreduce", world_size)
        with CommunicationOp(name=f"tree_ar_{executor}_rank{rank}") as op:
            op.tensor(dtype=dtype, shape=(tensor_size,))
            em = _Emit(op, executor, reduce_op, cuts)
            for c in range(num_channels):
                sig = c * 1000
                lo = c * tensor_size // num_channels
                n = (c + 1) * tensor_size // num_channels - lo
                with Stream("main" if num_channels == 1 else f"ch{c}"):
                    op.set_channel(c)
                    for k in range(log_n):
                        stride = 1 << k
                        partner = rank ^ stride
                        if rank & stride:
                            # child: announce, wait until the parent has consumed, leave
                            op.notify(signal_id=sig + rank, target_rank=partner)
                            op.wait_notify(signal_id=sig + partner, source_rank=partner)
                            break
                        if partner < world_size:
                            op.wait_notify(signal_id=sig + partner, source_rank=partner)
                            em.reduce(partner, lo, n)
                            op.notify(signal_id=sig + rank, target_rank=partner)
                    for k in range(log_n - 1, -1, -1):
                        stride = 1 << k
                        if rank % stride:
                            continue
                        partner = rank ^ stride
                        if rank & stride:
                            op.wait_notify(signal_id=sig + partner, source_rank=partner)
                            em.copy(partner, lo, n)
                            op.notify(signal_id=sig + rank, target_rank=partner)
                        elif partner < world_size:
                            op.notify(signal_id=sig + rank, target_rank=partner)
                            op.wait_notify(signal_id=sig + partner, source_rank=partner)
        g = op.get_graph()
        g.collective_type = "allreduce"
        return g
