"""Schedule templates named in the reference's ``ALGORITHMS`` table (algorithms/__init__.py:9-13)."""
from .base import CollectiveAlgorithm, pieces, ragged_cuts
from .ring import RingAllreduce
from .recursive_hd import RecursiveHalvingDoubling
from .tree import TreeAllreduce
from .selector import select_algorithm, select_algorithm_cost_based

ALGORITHMS = {"ring": RingAllreduce, "rhd": RecursiveHalvingDoubling, "tree": TreeAllreduce}

__all__ = ["CollectiveAlgorithm", "RingAllreduce", "RecursiveHalvingDoubling", "TreeAllreduce",
           "ALGORITHMS", "pieces", "ragged_cuts", "select_algorithm", "select_algorithm_cost_based"]
