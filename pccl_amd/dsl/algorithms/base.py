"""Common base of the schedule templates (interface of reference pccl/dsl/algorithms/base.py)."""
from __future__ import annotations

from typing import List, Optional, Sequence

from ..builder import CommunicationOp
from ..ir import Graph


class CollectiveAlgorithm:
    name: str = ""
    step_count: str = "unknown"
    bandwidth_optimal: bool = False

    def build_allreduce(self, rank, world_size, tensor_size, dtype="bfloat16", executor="tma",
                        num_channels=1, **ext) -> Graph:
        raise NotImplementedError

    def build_reduce_scatter(self, rank, world_size, tensor_size, dtype="bfloat16",
                             executor="tma", num_channels=1, **ext) -> Graph:
        raise NotImplementedError(f"{type(self).__name__} does not implement reduce_scatter")

    def build_allgather(self, rank, world_size, tensor_size, dtype="bfloat16", executor="tma",
                        num_channels=1, **ext) -> Graph:
        raise NotImplementedError(f"{type(self).__name__} does not implement allgather")

    def build_alltoall(self, rank, world_size, tensor_size, dtype="bfloat16", executor="tma",
                       num_channels=1, **ext) -> Graph:
        raise NotImplementedError(f"{type(self).__name__} does not implement alltoall")


def require_power_of_two(cls_name: str, world_size: int) -> int:
    if world_size <= 0 or world_size & (world_size - 1):
        raise ValueError(f"{cls_name} requires power-of-2 world_size, got {world_size}")
    return world_size.bit_length() - 1


def pieces(offset: int, count: int, cuts: Optional[Sequence[int]]) -> List[tuple]:
    """Split ``[offset, offset+count)`` at the absolute cut points that fall strictly inside it.

    ``cuts=None`` (the reference behaviour) yields the range itself.  Used by the ragged
    extension: the same cut list applied to every data op keeps all ranks' sub-op boundaries
    identical, so the ops stay position-aligned.
    """
    if not cuts:
        return [(offset, count)]
    inner = sorted(c for c in set(cuts) if offset < c < offset + count)
    edges = [offset] + inner + [offset + count]
    return [(a, b - a) for a, b in zip(edges[:-1], edges[1:])]


def ragged_cuts(tensor_size: int, num_pieces: int, seed: int = 0, vec_elems: int = 4) -> List[int]:
    """Cut points that make every piece start and end off a 16-byte boundary.

    Rule (published so results can be reproduced): cut ``i`` (1 <= i < num_pieces) sits at
    ``i*tensor_size//num_pieces`` moved down by ``1 + (lcg_i % (vec_elems-1))`` elements after
    rounding that base down to a multiple of ``vec_elems``, where ``lcg`` is the 31-bit
    generator ``x <- (1103515245*x + 12345) mod 2^31`` started at ``seed``.  Hence
    ``cut % vec_elems`` is in ``1..vec_elems-1``: no cut is a multiple of ``vec_elems`` elements
    (16 bytes for 4-byte types), and consecutive pieces have element counts that are generally
    not multiples of ``vec_elems`` either.
    """
    x = seed & 0x7FFFFFFF
    cuts = []
    for i in range(1, num_pieces):
        x = (1103515245 * x + 12345) & 0x7FFFFFFF
        base = (i * tensor_size // num_pieces) // vec_elems * vec_elems
        c = base - (1 + x % (vec_elems - 1))
        if 0 < c < tensor_size and (not cuts or c > cuts[-1]):
            cuts.append(c)
    return cuts


class _Emit:
    """Executor-dependent primitive names + optional ragged splitting of data ops."""

    def __init__(self, op: CommunicationOp, executor: str, reduce_op: str,
                 cuts: Optional[Sequence[int]]):
        self.op = op
        self.tma = executor == "tma"
        self.reduce_op = reduce_op
        self.cuts = cuts

    def reduce(self, source_rank: int, offset: int, count: int) -> None:
        fn = self.op.tma_reduce if self.tma else self.op.sm_reduce
        for off, n in pieces(offset, count, self.cuts):
            fn(reduce_op=self.reduce_op, source_rank=source_rank, src_offset=off,
               dst_offset=off, remote_offset=off, count=n)

    def copy(self, source_rank: int, offset: int, size: int) -> None:
        fn = self.op.tma_copy if self.tma else self.op.sm_copy
        for off, n in pieces(offset, size, self.cuts):
            fn(source_rank=source_rank, src_offset=off, dst_offset=off, size=n)
