"""Schedule emitter: builds per-rank primitive graphs and writes the JSON v2 files the executor loads."""
from .ir import Graph, Op, VALID_DTYPES, REFERENCE_DTYPES, DTYPE_BYTES
from .builder import CommunicationOp, Pipeline, Stream, build_graph
from .emit import Compiler, compile_to_json_string, compile_to_json_file
from .algorithms import (ALGORITHMS, CollectiveAlgorithm, RingAllreduce,
                         RecursiveHalvingDoubling, TreeAllreduce, ragged_cuts)

__all__ = ["Graph", "Op", "VALID_DTYPES", "REFERENCE_DTYPES", "DTYPE_BYTES", "CommunicationOp",
           "Stream", "Pipeline", "build_graph", "Compiler", "compile_to_json_string", "compile_to_json_file",
           "ALGORITHMS", "CollectiveAlgorithm", "RingAllreduce", "RecursiveHalvingDoubling",
           "TreeAllreduce", "ragged_cuts"]
