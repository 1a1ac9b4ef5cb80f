"""Builder front end: ``CommunicationOp`` / ``Stream`` with per-stream automatic chaining.

Call shape follows the reference builder (pccl/dsl/decorators.py:59-139,141-207,276-296) so that
schedule code written for it runs unchanged: ``with CommunicationOp(...) as op: op.tensor(...);
with Stream("ch0"): op.set_channel(0); op.notify(...); op.sm_reduce(...)``.
"""
from __future__ import annotations

from typing import Dict, List, Optional

from .ir import Graph, Op, VALID_DTYPES


class _StreamState:
    def __init__(self, name: str):
        self.name = name
        self.last: Optional[int] = None
        self.pending: List[int] = []


class Stream:
    """Context manager selecting the stream new ops are chained on."""
    _active_op: Optional["CommunicationOp"] = None

    def __init__(self, name: str):
        self.name = name
        self._prev: Optional[str] = None
        self._op: Optional[CommunicationOp] = None

    def __enter__(self) -> "Stream":
        if Stream._active_op is None:
            raise RuntimeError("Stream must be used within a CommunicationOp context")
        self._op = Stream._active_op
        self._prev = self._op._stream_name
        self._op._streams.setdefault(self.name, _StreamState(self.name))
        self._op._stream_name = self.name
        return self

    def __exit__(self, *exc) -> bool:
        self._op._stream_name = self._prev
        return False


class CommunicationOp:
    def __init__(self, name: str, device: object = None, auto_dependency: bool = True):
        self.name = name
        self.auto_dependency = auto_dependency
        self.graph = Graph(name)
        self._channel = 0
        self._streams: Dict[str, _StreamState] = {}
        self._stream_name: Optional[str] = None
        self._last: Optional[int] = None
        self._pending: List[int] = []

    def __enter__(self) -> "CommunicationOp":
        Stream._active_op = self
        return self

    def __exit__(self, exc_type, exc, tb) -> bool:
        Stream._active_op = None
        if exc_type is None:
            self._finalize()
        return False

    # -- configuration --------------------------------------------------------------------
    def tensor(self, dtype: str, shape: tuple) -> "CommunicationOp":
        if not isinstance(shape, tuple):
            raise ValueError(f"shape must be a tuple, got {type(shape)}")
        if str(dtype) not in VALID_DTYPES:
            raise ValueError(f"unsupported dtype '{dtype}', must be one of {sorted(VALID_DTYPES)}")
        self.graph.dtype, self.graph.shape = str(dtype), shape
        return self

    def set_channel(self, channel: int) -> "CommunicationOp":
        self._channel = channel
        return self

    # -- primitives -----------------------------------------------------------------------
    def _emit(self, primitive: str, params: dict) -> Op:
        deps: List[int] = []
        st = self._streams.get(self._stream_name) if self._stream_name else None
        if self.auto_dependency:
            if st is not None:
                deps.extend(st.pending)
                st.pending = []
                if st.last is not None:
                    deps.append(st.last)
            elif self._last is not None:
                deps.append(self._last)
        op = self.graph.add(primitive, params, self._channel, deps)
        if st is not None:
            st.last = op.uid
        else:
            self._last = op.uid
        return op

    def _reduce(self, prim, source_rank, src_offset, dst_offset, remote_offset, count, reduce_op):
        return self._emit(prim, {"reduce_op": reduce_op, "source_rank": source_rank,
                                 "src_offset": src_offset, "dst_offset": dst_offset,
                                 "remote_offset": remote_offset, "count": count})

    def _copy(self, prim, source_rank, src_offset, dst_offset, size):
        return self._emit(prim, {"source_rank": source_rank, "src_offset": src_offset,
                                 "dst_offset": dst_offset, "size": size})

    def sm_reduce(self, source_rank, src_offset, dst_offset, remote_offset, count,
                  reduce_op="sum"):
        return self._reduce("sm.reduce", source_rank, src_offset, dst_offset, remote_offset,
                            count, reduce_op)

    def tma_reduce(self, source_rank, src_offset, dst_offset, remote_offset, count,
                   reduce_op="sum"):
        return self._reduce("tma.reduce", source_rank, src_offset, dst_offset, remote_offset,
                            count, reduce_op)

    def sm_copy(self, source_rank, src_offset, dst_offset, size):
        return self._copy("sm.copy", source_rank, src_offset, dst_offset, size)

    def tma_copy(self, source_rank, src_offset, dst_offset, size):
        return self._copy("tma.copy", source_rank, src_offset, dst_offset, size)

    def notify(self, signal_id, target_rank):
        return self._emit("notify", {"signal_id": signal_id, "target_rank": target_rank})

    def wait_notify(self, signal_id, source_rank):
        return self._emit("wait_notify", {"signal_id": signal_id, "source_rank": source_rank})

    # -- cross-stream ordering ------------------------------------------------------------
    def wait(self, stream_name: str) -> None:
        target = self._streams.get(stream_name)
        if target is None:
            raise ValueError(f"Stream '{stream_name}' not found")
        if target.last is None:
            raise ValueError(f"Stream '{stream_name}' has no operations to wait for")
        self._defer(target.last)

    def wait_for(self, op: Op) -> None:
        if op is None or op.uid not in self.graph.ops:
            raise ValueError("Invalid node reference")
        self._defer(op.uid)

    def _defer(self, uid: int) -> None:
        st = self._streams.get(self._stream_name) if self._stream_name else None
        (st.pending if st is not None else self._pending).append(uid)

    # -- completion -----------------------------------------------------------------------
    def _finalize(self) -> None:
        if self.graph.is_empty():
            return
        for st in self._streams.values():
            if st.pending and st.last is not None:
                for d in st.pending:
                    self.graph.add_edge(d, st.last)
            st.pending = []
        if self._pending and self._last is not None:
            for d in self._pending:
                self.graph.add_edge(d, self._last)
        self._pending = []
        self.graph.relink()
        try:
            self.graph.validate()
        except ValueError as e:
            raise ValueError(f"Graph validation failed: {e}")

    def get_graph(self) -> Graph:
        return self.graph


def build_graph(name, builder_func, device=None) -> Graph:
    with CommunicationOp(name=name, device=device) as op:
        builder_func(op)
    return op.get_graph()


class _PipelineStage:
    def __init__(self, pipeline: "Pipeline"):
        self._pipeline = pipeline
        self._stream: Optional[Stream] = None

    def __enter__(self) -> "_PipelineStage":
        pipe = self._pipeline
        if pipe._op is None:
            raise RuntimeError("Pipeline.stage() must be used inside Pipeline.bind()")
        channel = pipe._iteration % pipe.depth
        pipe._iteration += 1
        pipe._op.set_channel(channel)
        self._stream = Stream(f"__pipe_ch{channel}")
        self._stream.__enter__()
        return self

    def __exit__(self, *exc) -> bool:
        if self._stream is not None:
            self._stream.__exit__(*exc)
        return False


class _PipelineBinding:
    def __init__(self, pipeline: "Pipeline", op: CommunicationOp):
        self._pipeline, self._target = pipeline, op

    def __enter__(self) -> "Pipeline":
        self._pipeline._op = self._target
        self._pipeline._iteration = 0
        return self._pipeline

    def __exit__(self, *exc) -> bool:
        self._pipeline._op = None
        return False


class Pipeline:
    """Step-level pipelining over channels (reference pccl/dsl/pipeline.py:64-88): the k-th
    ``stage()`` of a bound pipeline puts its ops on channel ``k % depth`` and on the stream
    ``__pipe_ch<channel>``, so stages on one channel run in order and different channels are
    independent of each other."""

    def __init__(self, depth: int = 2):
        if depth < 1:
            raise ValueError(f"Pipeline depth must be >= 1, got {depth}")
        self.depth = depth
        self._op: Optional[CommunicationOp] = None
        self._iteration = 0

    def bind(self, op: CommunicationOp) -> _PipelineBinding:
        return _PipelineBinding(self, op)

    def stage(self) -> _PipelineStage:
        return _PipelineStage(self)
