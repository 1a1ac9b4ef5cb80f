"""Choice of the allreduce schedule for a world size and message size.

Reference: pccl/dsl/algorithms/selector.py.  ``select_algorithm`` is the size heuristic (ring for
large messages and for world sizes that are not powers of two, recursive halving-doubling for
messages under 1 MiB on four or more ranks); ``select_algorithm_cost_based`` builds every
candidate for the rank and keeps the one whose graph has the shortest critical path under a
device profile (``channelize.critical_path_cost_us``).
"""
from __future__ import annotations

from ..channelize import H100_PROFILE, DeviceProfile, critical_path_cost_us
from .base import CollectiveAlgorithm
from .recursive_hd import RecursiveHalvingDoubling
from .ring import RingAllreduce
from .tree import TreeAllreduce


def _power_of_two(n: int) -> bool:
    return n > 0 and (n & (n - 1)) == 0


def select_algorithm(world_size: int, data_bytes: int, topology: object = None,
                     device: DeviceProfile = H100_PROFILE) -> CollectiveAlgorithm:
    if not _power_of_two(world_size) or world_size <= 2:
        return RingAllreduce()
    if data_bytes >= 1024 * 1024:
        return RingAllreduce()
    return RecursiveHalvingDoubling()      # world_size >= 4 here


def graph_cost_us(graph, device: DeviceProfile, data_bytes: int) -> float:
    """Critical path of one rank's graph, every data op priced at `data_bytes`."""
    graph.relink()
    order = list(graph.ops.values())
    index = {o.uid: i for i, o in enumerate(order)}
    nodes = [(o.primitive, o.channel) for o in order]
    edges = [(index[o.uid], index[n]) for o in order for n in o.nexts]
    return critical_path_cost_us(nodes, edges, device, data_bytes)


def select_algorithm_cost_based(rank: int, world_size: int, tensor_size: int, data_bytes: int,
                                topology: object = None, device: DeviceProfile = H100_PROFILE,
                                dtype: str = "bfloat16", executor: str = "tma") -> CollectiveAlgorithm:
    candidates = [RingAllreduce()]
    if _power_of_two(world_size) and world_size >= 2:
        candidates += [RecursiveHalvingDoubling(), TreeAllreduce()]
    best, best_cost = candidates[0], float("inf")
    for alg in candidates:
        try:
            g = alg.build_allreduce(rank=rank, world_size=world_size, tensor_size=tensor_size,
                                    dtype=dtype, executor=executor)
        except Exception:
            continue
        cost = graph_cost_us(g, device, data_bytes)
        if cost < best_cost:
            best, best_cost = alg, cost
    return best
