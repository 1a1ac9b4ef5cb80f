"""pccl_amd — MI355X-native executor for PCCL's SM reduce/copy data path, plus the schedule emitter.

``pccl_amd.dsl`` builds per-rank graphs and writes the JSON v2 files; ``pccl_amd.engine`` registers
and executes them on one GPU with the R ranks held as virtual ranks.  The executor is the HIP
library ``pccl_amd/lib/libpccl_hip.so`` (C ABI in ``include/pccl_hip.h``); importing
``pccl_amd.engine`` without it raises.
"""
__version__ = "0.1.0"

from . import dsl  # noqa: F401
from .dsl import (ALGORITHMS, CommunicationOp, Compiler, RecursiveHalvingDoubling, RingAllreduce,  # noqa: F401
                  Stream, TreeAllreduce, build_graph, compile_to_json_file, compile_to_json_string)
