"""ctypes front end of the CPU oracle — TEST INFRASTRUCTURE ONLY (tests, smoke check, CPU baseline).

Graph loading here is deliberately independent of the product's C++ loader: it reads the JSON v2
document with the standard library and maps fields exactly as the reference's channel parsers do
(csrc/plugins/cuda/channels/sm_channel.h:26-96, tma_channel.h:27-81;
csrc/engine/graph_builder.cc:12-107), so that a loader bug in the product cannot hide behind an
identical bug in the checker.
"""
from __future__ import annotations

import ctypes
import json
import os
from typing import List, Sequence

import numpy as np

from . import build as _build

DT = {"float32": 0, "float16": 1, "bfloat16": 2, "float8_e4m3": 3, "float8_e5m2": 4, "int32": 5}
ESIZE = {0: 4, 1: 2, 2: 2, 3: 1, 4: 1, 5: 4}
RED = {"sum": 0, "max": 1, "min": 2}
K_NOOP, K_REDUCE, K_COPY, K_NOTIFY, K_WAIT = range(5)
MAX_NEXT = 8


class OracleOp(ctypes.Structure):
    _fields_ = [(n, ctypes.c_int32) for n in
                ("kind", "index", "channel", "peer", "off0", "off1", "off2", "size", "redop",
                 "ndeps", "nnext")] + [("next", ctypes.c_int32 * MAX_NEXT)]


class OracleStats(ctypes.Structure):
    _fields_ = [("ops_executed", ctypes.c_int64), ("data_ops", ctypes.c_int64),
                ("bytes", ctypes.c_int64), ("deadlocked", ctypes.c_int32),
                ("residual", ctypes.c_int32)]


_lib = None


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        path = _build.OUT
        if not os.path.exists(path):
            _build.build()
        _lib = ctypes.CDLL(path)
        _lib.pccl_oracle_last_error.restype = ctypes.c_char_p
        assert _lib.pccl_oracle_sizeof_op() == ctypes.sizeof(OracleOp)
    return _lib


class OracleError(RuntimeError):
    pass


class Graph:
    """One rank's parsed graph."""

    def __init__(self, doc: dict):
        if "operations" not in doc:
            raise OracleError("graph has no 'operations'")
        info = doc.get("tensor_info", {})
        self.dtype_name = info.get("dtype", "float32")
        self.shape = info.get("shape", [])
        self.collective_type = doc.get("collective_type", "")
        ops = doc["operations"]
        self.table = (OracleOp * max(len(ops), 1))()
        self.n = len(ops)
        has_data = False
        for pos, op in enumerate(ops):
            for key in ("index", "executor", "primitive"):
                if key not in op:
                    raise OracleError(f"operation {pos} lacks '{key}'")
            o = self.table[pos]
            prim, p = op["primitive"], op.get("params", {})
            o.index, o.channel = op["index"], op.get("channel", 0)
            o.ndeps = len(op.get("dependencies", []))
            nxt = op.get("next_ops", [])[:MAX_NEXT]
            o.nnext = len(nxt)
            for k, v in enumerate(nxt):
                o.next[k] = v
            if prim in ("sm.reduce", "tma.reduce"):
                has_data = True
                o.kind = K_REDUCE
                o.peer = p.get("source_rank", p.get("target_rank", 0))
                o.off0, o.off1, o.off2 = p["remote_offset"], p["src_offset"], p["dst_offset"]
                o.size = p["count"]
                red = p.get("reduce_op", "sum")
                if red not in RED:
                    raise OracleError(f"reduce_op '{red}' not supported")
                o.redop = RED[red]
            elif prim in ("sm.copy", "tma.copy"):
                has_data = True
                o.kind = K_COPY
                o.peer = p.get("source_rank", p.get("target_rank", 0))
                o.off0, o.off1, o.size = p["src_offset"], p["dst_offset"], p["size"]
            elif prim in ("notify", "sm.notify"):
                o.kind, o.peer, o.off0 = K_NOTIFY, p["target_rank"], p["signal_id"]
            elif prim in ("wait_notify", "sm.wait_notify"):
                o.kind, o.peer, o.off0 = K_WAIT, p["source_rank"], p["signal_id"]
            elif prim == "noop":
                o.kind = K_NOOP
            else:
                raise OracleError(f"unknown primitive '{prim}'")
        if has_data and self.dtype_name not in DT:
            raise OracleError(f"Unsupported dtype '{self.dtype_name}'")
        self.dtype = DT.get(self.dtype_name, 0)

    @classmethod
    def from_file(cls, path: str) -> "Graph":
        with open(path) as f:
            return cls(json.load(f))


NUM_SIGNALS = 4096    # semaphores per rank (include/common/config.h:24)


def new_signals(world: int) -> np.ndarray:
    """The semaphore state of an engine with ``world`` ranks, all zero: pass it to consecutive
    ``run`` calls to carry counts from one execution into the next (csrc/engine_c.cc:576-593)."""
    return np.zeros((world, NUM_SIGNALS), dtype=np.int32)


def run(graphs: Sequence[Graph], bufs: List[np.ndarray], sched_seed: int = 0,
        threads: int = 0, signals: np.ndarray = None) -> OracleStats:
    """Execute the R graphs in place on ``bufs`` (one contiguous array per rank, raw storage:
    float32/int32 as themselves, float16/bfloat16 as uint16 bit patterns).  ``signals`` (from
    ``new_signals``) is the semaphore state to start from, updated in place; None starts from zero."""
    L = lib()
    R = len(graphs)
    dtype = graphs[0].dtype
    es = ESIZE[dtype]
    nelems = bufs[0].nbytes // es
    for b in bufs:
        assert b.flags["C_CONTIGUOUS"] and b.nbytes // es == nelems
    nops = (ctypes.c_int32 * R)(*[g.n for g in graphs])
    tabs = (ctypes.POINTER(OracleOp) * R)(*[ctypes.cast(g.table, ctypes.POINTER(OracleOp))
                                             for g in graphs])
    ptrs = (ctypes.c_void_p * R)(*[b.ctypes.data for b in bufs])
    st = OracleStats()
    if signals is not None:
        assert signals.dtype == np.int32 and signals.shape == (R, NUM_SIGNALS) and signals.flags["C_CONTIGUOUS"]
    rc = L.pccl_oracle_run_carry(R, nops, tabs, dtype, ptrs, ctypes.c_int64(nelems),
                                 ctypes.c_uint32(sched_seed), threads,
                                 ctypes.c_void_p(signals.ctypes.data if signals is not None else None), ctypes.byref(st))
    if rc != 0:
        raise OracleError(L.pccl_oracle_last_error().decode())
    return st


def reduce(dtype: str, redop: str, a: np.ndarray, b: np.ndarray) -> np.ndarray:
    L = lib()
    c = np.empty_like(a)
    rc = L.pccl_oracle_reduce(DT[dtype], RED[redop], ctypes.c_void_p(a.ctypes.data),
                              ctypes.c_void_p(b.ctypes.data), ctypes.c_void_p(c.ctypes.data),
                              ctypes.c_int64(a.nbytes // ESIZE[DT[dtype]]))
    if rc != 0:
        raise OracleError(L.pccl_oracle_last_error().decode())
    return c
