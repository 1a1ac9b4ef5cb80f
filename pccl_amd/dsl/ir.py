"""Graph IR for the schedule emitter: one flat record type per primitive, plus the DAG container.

This is a from-scratch emitter for the reference's JSON v2 wire format (the format the executor
consumes), not a re-implementation of the reference DSL stack.  What has to agree with the
reference is the emitted document:

* primitive / executor strings            (reference pccl/dsl/nodes.py:23-52, codegen/mapping.py:7-14)
* per-primitive ``params`` keys and order (reference pccl/dsl/nodes.py:154-159,181-185,388-429)
* ``index`` = position in a Kahn topological order with a FIFO ready queue seeded in insertion
  order                                   (reference pccl/dsl/graph.py:203-218)
* ``next_ops`` = dependents in insertion order (reference pccl/dsl/passes/dependency_analysis.py:48-66)

Extensions beyond the reference (it rejects them): dtype ``int32`` and an honoured ``reduce_op``
of ``max`` / ``min``.
"""
from __future__ import annotations

from collections import deque
from dataclasses import dataclass, field
from typing import Dict, List, Optional, Tuple

# primitive name -> executor string written to JSON
EXECUTOR_OF = {
    "sm.reduce": "cuda_sm", "sm.copy": "cuda_sm",
    "tma.reduce": "cuda_tma", "tma.copy": "cuda_tma",
    "notify": "cuda_sm", "wait_notify": "cuda_sm", "noop": "cuda_sm",
}

REFERENCE_DTYPES = ("float32", "float16", "bfloat16", "float8_e4m3", "float8_e5m2")
EXTENSION_DTYPES = ("int32",)
VALID_DTYPES = REFERENCE_DTYPES + EXTENSION_DTYPES
REDUCE_OPS = ("sum", "max", "min", "avg")

DTYPE_BYTES = {"float32": 4, "float16": 2, "bfloat16": 2, "float8_e4m3": 1, "float8_e5m2": 1,
               "int32": 4}


@dataclass
class Op:
    """One primitive.  ``params`` keeps the key order the JSON must have."""
    uid: int
    primitive: str
    params: Dict[str, object]
    channel: int = 0
    deps: List[int] = field(default_factory=list)
    nexts: List[int] = field(default_factory=list)

    @property
    def executor(self) -> str:
        return EXECUTOR_OF[self.primitive]

    @property
    def is_data(self) -> bool:
        return self.primitive.endswith((".reduce", ".copy"))

    def validate(self) -> None:
        p = self.params
        if self.primitive.endswith(".reduce"):
            if p["reduce_op"] not in REDUCE_OPS:
                raise ValueError(f"{self.primitive}: invalid reduce_op '{p['reduce_op']}'")
            if p["source_rank"] < 0:
                raise ValueError(f"{self.primitive}: source_rank must be non-negative")
            if p["count"] < 0:
                raise ValueError(f"{self.primitive}: count must be non-negative")
        elif self.primitive.endswith(".copy"):
            if p["source_rank"] < 0:
                raise ValueError(f"{self.primitive}: source_rank must be non-negative")
            if p["size"] < 0:
                raise ValueError(f"{self.primitive}: size must be non-negative")
        elif self.primitive == "notify":
            if p["target_rank"] < 0:
                raise ValueError("notify: target_rank must be non-negative")
        elif self.primitive == "wait_notify":
            if p["source_rank"] < 0:
                raise ValueError("wait_notify: source_rank must be non-negative")


class Graph:
    """Insertion-ordered DAG of :class:`Op` for one rank."""

    def __init__(self, name: str = "unnamed_graph"):
        self.name = name
        self.ops: Dict[int, Op] = {}
        self.dtype: Optional[str] = None
        self.shape: Optional[Tuple[int, ...]] = None
        self.collective_type: str = ""
        self._next_uid = 0

    # -- construction ---------------------------------------------------------------------
    def add(self, primitive: str, params: Dict[str, object], channel: int,
            deps: List[int]) -> Op:
        if primitive not in EXECUTOR_OF:
            raise ValueError(f"unknown primitive '{primitive}'")
        op = Op(self._next_uid, primitive, params, channel, [])
        self._next_uid += 1
        for d in deps:
            if d not in self.ops:
                raise KeyError(f"dependency {d} is not in the graph")
            if d not in op.deps:
                op.deps.append(d)
        self.ops[op.uid] = op
        return op

    def add_edge(self, src: int, dst: int) -> None:
        if src == dst:
            raise ValueError("self-loop")
        if src not in self.ops[dst].deps:
            self.ops[dst].deps.append(src)

    # -- queries --------------------------------------------------------------------------
    def size(self) -> int:
        return len(self.ops)

    def is_empty(self) -> bool:
        return not self.ops

    def count(self, primitive_suffix: str) -> int:
        return sum(1 for o in self.ops.values() if o.primitive.endswith(primitive_suffix))

    # -- passes ---------------------------------------------------------------------------
    def relink(self) -> None:
        """Rebuild ``nexts`` from ``deps``: dependents listed in insertion order."""
        for o in self.ops.values():
            o.nexts = []
        for o in self.ops.values():
            for d in o.deps:
                if o.uid not in self.ops[d].nexts:
                    self.ops[d].nexts.append(o.uid)

    def eliminate_dead(self) -> int:
        """Drop ops from which no exit op and no notify is reachable (forward)."""
        keep = set()
        stack = [o.uid for o in self.ops.values() if not o.nexts or o.primitive == "notify"]
        while stack:
            u = stack.pop()
            if u in keep:
                continue
            keep.add(u)
            stack.extend(self.ops[u].deps)
        dead = [u for u in self.ops if u not in keep]
        for u in dead:
            del self.ops[u]
        for o in self.ops.values():
            o.deps = [d for d in o.deps if d in self.ops]
        self.relink()
        return len(dead)

    def topo_order(self) -> List[Op]:
        indeg = {u: len(o.deps) for u, o in self.ops.items()}
        ready = deque(u for u, d in indeg.items() if d == 0)
        out: List[Op] = []
        while ready:
            u = ready.popleft()
            out.append(self.ops[u])
            for v in self.ops[u].nexts:
                indeg[v] -= 1
                if indeg[v] == 0:
                    ready.append(v)
        if len(out) != len(self.ops):
            raise ValueError("Graph contains a cycle")
        return out

    def validate(self) -> None:
        if not self.ops:
            raise ValueError("Graph is empty (no nodes)")
        for o in self.ops.values():
            o.validate()
        self.topo_order()

    # -- emission -------------------------------------------------------------------------
    def to_runtime_dict(self) -> Dict[str, object]:
        """The JSON v2 document (reference pccl/dsl/codegen/json_generator.py:46-83)."""
        self.validate()
        order = self.topo_order()
        index = {o.uid: i for i, o in enumerate(order)}
        doc: Dict[str, object] = {"version": 2}
        if self.dtype is not None:
            doc["tensor_info"] = {"dtype": self.dtype, "shape": list(self.shape)}
        if self.collective_type:
            doc["collective_type"] = self.collective_type
        executors: Dict[str, bool] = {}
        operations = []
        for o in order:
            executors[o.executor] = True
            operations.append({
                "index": index[o.uid],
                "executor": o.executor,
                "primitive": o.primitive,
                "channel": o.channel,
                "dependencies": [index[d] for d in o.deps],
                "next_ops": [index[n] for n in o.nexts],
                "params": dict(o.params),
            })
        doc["executors"] = list(executors)
        doc["operations"] = operations
        return doc
