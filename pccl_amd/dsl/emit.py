"""Compile a :class:`Graph` to the JSON v2 text the executor loads.

Default pipeline = relink -> dead-op elimination -> relink -> emit, the observable effect of the
reference's ``Compiler().compile`` with its defaults (pccl/dsl/compiler.py:33-54);
``enable_channelize`` adds the channelisation pass between the two, as there.
"""
from __future__ import annotations

import json
from typing import Optional

from .channelize import H100_PROFILE, ChannelizePass, DeviceProfile
from .ir import Graph


class Compiler:
    def __init__(self, enable_dce: bool = True, enable_channelize: bool = False, num_channels: int = 2,
                 device_profile: Optional[DeviceProfile] = None):
        self.enable_dce = enable_dce
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
