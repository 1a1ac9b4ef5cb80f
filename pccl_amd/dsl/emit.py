"""Compile a :class:`Graph` to the JSON v2 text the executor loads.

Default pipeline = relink -> dead-op elimination -> relink -> emit, the observable effect of the
reference's ``Compiler().compile`` with its defaults (pccl/dsl/compiler.py:33-54);
``enable_channelize`` adds the channelisation pass between the two, as there.

``enable_superopt`` applies the executor upgrades of the reference's superoptimisation pass
(pccl/dsl/superopt/pass_.py:76-87, enumerator.py:44-47: every ``sm.copy`` / ``sm.reduce`` becomes
``tma.copy`` / ``tma.reduce``), which is what the reference's own tests pin of that pass
(tests/test_superopt.py:813-851: no ``cuda_sm`` data executor survives, the document keeps its
shape).  The e-graph rewriting that follows there (SMT-discovered rules, needs z3) is not
reproduced; for the templates it keeps the chains as they are.  This executor runs ``tma.*`` as
the SM ops, so the pass changes names, not results.
"""
from __future__ import annotations

import json
from typing import Optional

from .channelize import H100_PROFILE, ChannelizePass, DeviceProfile
from .ir import Graph


EXECUTOR_UPGRADES = {"sm.copy": "tma.copy", "sm.reduce": "tma.reduce"}


class Compiler:
    def __init__(self, enable_dce: bool = True, enable_superopt: bool = False, enable_channelize: bool = False,
                 num_channels: int = 2, gpu_profile: str = "h100", data_size_hint: int = 0, topology: object = None,
                 device_profile: Optional[DeviceProfile] = None):
        # gpu_profile, data_size_hint, topology: knobs of the reference's e-graph search, accepted and unused
        self.enable_dce = enable_dce
        self.enable_superopt = enable_superopt
        self.enable_channelize = enable_channelize
        self.num_channels = num_channels
        self.device_profile = device_profile

    def compile(self, graph: Graph) -> Graph:
        if graph.is_empty():
            raise ValueError("Cannot analyze empty graph")
        graph.relink()
        graph.validate()
        if self.enable_dce:
            graph.eliminate_dead()
        if self.enable_superopt:
            for op in graph.ops.values():
                if op.primitive in EXECUTOR_UPGRADES:
                    op.primitive = EXECUTOR_UPGRADES[op.primitive]
        if self.enable_channelize:   # reference compiler.py:51-52 (which always uses its default profile)
            ChannelizePass(num_channels=self.num_channels,
                           profile=self.device_profile or H100_PROFILE).run(graph)
        graph.relink()
        return graph

    def compile_to_dict(self, graph: Graph) -> dict:
        return self.compile(graph).to_runtime_dict()

    def compile_to_json(self, graph: Graph, output_file: Optional[str] = None,
                        indent: int = 2) -> str:
        text = json.dumps(self.compile_to_dict(graph), indent=indent)
        if output_file:
            with open(output_file, "w") as f:
                f.write(text)
        return text


def compile_to_json_string(graph: Graph, indent: int = 2) -> str:
    return Compiler().compile_to_json(graph, None, indent)


def compile_to_json_file(graph: Graph, output_file: str, indent: int = 2) -> str:
    return Compiler().compile_to_json(graph, output_file, indent)
