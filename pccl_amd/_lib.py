"""ctypes binding of libpccl_hip.so (the C ABI declared in include/pccl_hip.h).

There is no fallback: if the library is missing the import of anything that needs it raises.
"""
from __future__ import annotations

import ctypes
import os

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "lib", "libpccl_hip.so")

MAX_VRANKS = 64
MAX_CHANNELS = 8

OK, ERR_INVALID, ERR_NOT_FOUND, ERR_PARSE, ERR_LINK, ERR_HIP, ERR_UNSUPPORTED, ERR_NOT_A_GRAPH = 0, -1, -2, -3, -4, -5, -6, -7

DTYPE_ID = {"float32": 0, "float16": 1, "bfloat16": 2, "float8_e4m3": 3, "float8_e5m2": 4, "int32": 5}
REDOP_ID = {"sum": 0, "max": 1, "min": 2}


class Trigger(ctypes.Structure):
    _fields_ = [("primitive_type", ctypes.c_int8), ("redop", ctypes.c_int8), ("pad_", ctypes.c_int8 * 2),
                ("op_index", ctypes.c_int32), ("peer_rank", ctypes.c_int32), ("offset_0", ctypes.c_int32),
                ("offset_1", ctypes.c_int32), ("offset_2", ctypes.c_int32), ("size", ctypes.c_int32),
                ("reserved_", ctypes.c_int32)]


class PrimitiveMeta(ctypes.Structure):
    _fields_ = [("op_seq_index", ctypes.c_int32), ("num_next_ops", ctypes.c_int32),
                ("num_dependencies", ctypes.c_int32), ("next_primitive_index", ctypes.c_int32 * 8),
                ("device_type", ctypes.c_int32), ("channel", ctypes.c_int32), ("params", ctypes.c_uint64 * 4)]


class FusedStep(ctypes.Structure):
    _fields_ = [("primitive_type", ctypes.c_int8), ("pad_", ctypes.c_int8 * 3), ("peer_rank", ctypes.c_int32),
                ("offset_0", ctypes.c_int32), ("offset_1", ctypes.c_int32), ("offset_2", ctypes.c_int32),
                ("size", ctypes.c_int32), ("notify_signal_id", ctypes.c_int32),
                ("notify_peer_rank", ctypes.c_int32), ("wait_signal_id", ctypes.c_int32),
                ("wait_peer_rank", ctypes.c_int32), ("has_notify", ctypes.c_uint8), ("has_wait", ctypes.c_uint8),
                ("pad2_", ctypes.c_uint8 * 2)]


class ProgramInfo(ctypes.Structure):
    _fields_ = [("num_vranks", ctypes.c_int32), ("dtype", ctypes.c_int32), ("num_ops", ctypes.c_int32),
                ("num_data_ops", ctypes.c_int32), ("num_levels", ctypes.c_int32),
                ("position_aligned", ctypes.c_int32), ("num_segments", ctypes.c_int32),
                ("residual_signals", ctypes.c_int32), ("buffer_elems", ctypes.c_int64),
                ("algorithmic_bytes", ctypes.c_int64), ("column_load_bytes", ctypes.c_int64),
                ("column_store_bytes", ctypes.c_int64), ("num_items", ctypes.c_int32),
                ("num_gather_copies", ctypes.c_int32), ("staged_load_bytes", ctypes.c_int64),
                ("staged_store_bytes", ctypes.c_int64), ("race_checked", ctypes.c_int32),
                ("order_checked", ctypes.c_int32), ("chain_segments", ctypes.c_int32),
                ("staged_chain_segments", ctypes.c_int32)]

    def as_dict(self):
        return {n: getattr(self, n) for n, _ in self._fields_ if not n.endswith("_")}


class ColumnSegment(ctypes.Structure):
    _fields_ = [("start", ctypes.c_int64), ("end", ctypes.c_int64), ("prog_start", ctypes.c_int32),
                ("prog_len", ctypes.c_int32), ("pre_start", ctypes.c_int32), ("pre_words", ctypes.c_int32),
                ("bcast_mask", ctypes.c_uint64)]


class LinkedOp(ctypes.Structure):
    _fields_ = [(n, ctypes.c_int32) for n in ("rank", "channel", "op_index", "is_reduce", "redop",
                                              "peer_rank", "level", "num_deps")] + \
               [(n, ctypes.c_int64) for n in ("offset_0", "offset_1", "offset_2", "size")] + \
               [("deps", ctypes.c_int32 * 8)]


class PcclError(RuntimeError):
    def __init__(self, code: int, message: str):
        super().__init__(message)
        self.code = code


_lib = None

# every symbol include/pccl_hip.h declares
EXPORTS = [
    "pccl_graph_load_file", "pccl_graph_load_json", "pccl_graph_from_triggers", "pccl_graph_free",
    "pccl_graph_num_ops", "pccl_graph_dtype", "pccl_graph_tensor_elems", "pccl_graph_collective_type",
    "pccl_graph_get_triggers", "pccl_graph_get_meta", "pccl_graph_fused_steps", "pccl_program_link",
    "pccl_program_link_carried", "pccl_program_get_signals",
    "pccl_program_free", "pccl_program_get_info", "pccl_program_get_ops", "pccl_program_get_column",
    "pccl_hip_create",
    "pccl_hip_destroy", "pccl_hip_register_file", "pccl_hip_register_json", "pccl_hip_register_triggers",
    "pccl_hip_set_option", "pccl_hip_get_option", "pccl_hip_execute", "pccl_hip_execute_inplace", "pccl_hip_execute_inplace_static", "pccl_hip_sync",
    "pccl_hip_reset_signals", "pccl_hip_op_info", "pccl_hip_last_kernel_ms", "pccl_hip_reduce",
    "pccl_hip_copy", "pccl_hip_last_error", "pccl_hip_version",
]


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise ImportError(
            f"{LIB_PATH} is missing: build it with `python -m pccl_amd.build` (hipcc, gfx950). "
            "The executor has no CPU or PyTorch fallback.")
    # PyTorch-ROCm ships its own HIP runtime (libamdhip64.so.7).  It must be in the process before
    # this library is, so that the dynamic loader binds this library to that same runtime; loaded
    # the other way round the process ends up with two HIP runtimes and neither sees the other's
    # device state.
    import torch  # noqa: F401
    L = ctypes.CDLL(LIB_PATH)
    vp, cp, i32, i64, sz = ctypes.c_void_p, ctypes.c_char_p, ctypes.c_int, ctypes.c_int64, ctypes.c_size_t
    P = ctypes.POINTER
    sigs = {
        "pccl_graph_load_file": (i32, [cp, P(vp)]),
        "pccl_graph_load_json": (i32, [cp, sz, P(vp)]),
        "pccl_graph_from_triggers": (i32, [P(Trigger), P(PrimitiveMeta), i32, cp, P(vp)]),
        "pccl_graph_free": (None, [vp]),
        "pccl_graph_num_ops": (i32, [vp]),
        "pccl_graph_dtype": (i32, [vp]),
        "pccl_graph_tensor_elems": (i64, [vp]),
        "pccl_graph_collective_type": (cp, [vp]),
        "pccl_graph_get_triggers": (i32, [vp, P(Trigger), i32]),
        "pccl_graph_get_meta": (i32, [vp, P(PrimitiveMeta), i32]),
        "pccl_graph_fused_steps": (i32, [vp, P(FusedStep), i32, P(ctypes.c_int), P(ctypes.c_int)]),
        "pccl_program_link": (i32, [P(vp), i32, P(vp)]),
        "pccl_program_link_carried": (i32, [P(vp), i32, P(ctypes.c_int32), i32, P(vp)]),
        "pccl_program_get_signals": (i32, [vp, P(ctypes.c_int32), i32]),
        "pccl_program_free": (None, [vp]),
        "pccl_program_get_info": (i32, [vp, P(ProgramInfo)]),
        "pccl_program_get_ops": (i32, [vp, P(LinkedOp), i32]),
        "pccl_program_get_column": (i32, [vp, i32, P(ColumnSegment), i32, P(ctypes.c_int), P(ctypes.c_uint64), i32,
                                          P(ctypes.c_int), P(ctypes.c_uint64), i32, P(ctypes.c_int), P(i64), P(i64)]),
        "pccl_hip_create": (i32, [P(vp), i32, i32]),
        "pccl_hip_destroy": (i32, [vp]),
        "pccl_hip_register_file": (i32, [vp, cp, i32, cp]),
        "pccl_hip_register_json": (i32, [vp, cp, i32, cp, sz]),
        "pccl_hip_register_triggers": (i32, [vp, cp, i32, P(Trigger), P(PrimitiveMeta), i32, cp]),
        "pccl_hip_set_option": (i32, [vp, cp, cp]),
        "pccl_hip_get_option": (i32, [vp, cp, ctypes.c_char_p, ctypes.c_size_t]),
        "pccl_hip_execute": (i32, [vp, cp, P(vp), P(vp), sz, sz, vp, i32]),
        "pccl_hip_execute_inplace": (i32, [vp, cp, P(vp), sz, vp, i32]),
        "pccl_hip_execute_inplace_static": (i32, [vp, cp, P(vp), sz, vp, i32]),
        "pccl_hip_sync": (i32, [vp, cp]),
        "pccl_hip_reset_signals": (i32, [vp, cp]),
        "pccl_hip_op_info": (i32, [vp, cp, P(ProgramInfo)]),
        "pccl_hip_last_kernel_ms": (i32, [vp, cp, P(ctypes.c_float)]),
        "pccl_hip_reduce": (i32, [i32, i32, vp, vp, vp, sz, vp]),
        "pccl_hip_copy": (i32, [i32, vp, vp, sz, vp]),
        "pccl_hip_last_error": (cp, []),
        "pccl_hip_version": (cp, []),
    }
    for name, (res, args) in sigs.items():
        fn = getattr(L, name)
        fn.restype, fn.argtypes = res, args
    _lib = L
    return L


def check(rc: int) -> int:
    if rc < 0:
        raise PcclError(rc, lib().pccl_hip_last_error().decode(errors="replace"))
    return rc


# -- host-only helpers (no GPU needed) ---------------------------------------------------------

class HostGraph:
    """One rank's loaded graph (host side only)."""

    def __init__(self, handle):
        self._h = handle

    @classmethod
    def from_json(cls, text: str) -> "HostGraph":
        h = ctypes.c_void_p()
        data = text.encode()
        check(lib().pccl_graph_load_json(data, len(data), ctypes.byref(h)))
        return cls(h)

    @classmethod
    def from_file(cls, path: str) -> "HostGraph":
        h = ctypes.c_void_p()
        check(lib().pccl_graph_load_file(path.encode(), ctypes.byref(h)))
        return cls(h)

    @classmethod
    def from_triggers(cls, triggers, meta, collective_type: str = "") -> "HostGraph":
        h = ctypes.c_void_p()
        n = len(triggers)
        check(lib().pccl_graph_from_triggers(triggers, meta, n, collective_type.encode(), ctypes.byref(h)))
        return cls(h)

    def __del__(self):
        if getattr(self, "_h", None) and _lib is not None:
            _lib.pccl_graph_free(self._h)
            self._h = None

    @property
    def num_ops(self) -> int:
        return lib().pccl_graph_num_ops(self._h)

    @property
    def dtype(self) -> int:
        return lib().pccl_graph_dtype(self._h)

    @property
    def tensor_elems(self) -> int:
        return lib().pccl_graph_tensor_elems(self._h)

    @property
    def collective_type(self) -> str:
        return lib().pccl_graph_collective_type(self._h).decode()

    def triggers(self):
        n = self.num_ops
        arr = (Trigger * max(n, 1))()
        check(lib().pccl_graph_get_triggers(self._h, arr, n))
        return arr, n

    def meta(self):
        n = self.num_ops
        arr = (PrimitiveMeta * max(n, 1))()
        check(lib().pccl_graph_get_meta(self._h, arr, n))
        return arr, n

    def fused_steps(self):
        """Returns (steps, channel_offsets) or raises PcclError(ERR_UNSUPPORTED)."""
        steps = (FusedStep * 128)()
        offs = (ctypes.c_int * (MAX_CHANNELS + 1))()
        nch = ctypes.c_int()
        n = check(lib().pccl_graph_fused_steps(self._h, steps, 128, offs, ctypes.byref(nch)))
        return [steps[i] for i in range(n)], [offs[i] for i in range(nch.value + 1)]


class HostProgram:
    """R graphs linked into one program (host side only)."""

    def __init__(self, graphs, carried=None):
        """``carried``: ``{(rank, signal_id): count}`` left by earlier executions (default: none)."""
        arr = (ctypes.c_void_p * len(graphs))(*[g._h for g in graphs])
        h = ctypes.c_void_p()
        flat = [v for (rank, sid), count in sorted((carried or {}).items()) for v in (rank, sid, count)]
        trip = (ctypes.c_int32 * max(len(flat), 1))(*flat)
        check(lib().pccl_program_link_carried(arr, len(graphs), trip, len(flat) // 3, ctypes.byref(h)))
        self._h = h
        self._graphs = graphs

    def signals(self) -> dict:
        """``{(rank, signal_id): (notifies, waits)}`` of one execution."""
        L = lib()
        n = L.pccl_program_get_signals(self._h, None, 0)
        buf = (ctypes.c_int32 * max(4 * n, 1))()
        L.pccl_program_get_signals(self._h, buf, n)
        return {(buf[4 * i], buf[4 * i + 1]): (buf[4 * i + 2], buf[4 * i + 3]) for i in range(n)}

    def __del__(self):
        if getattr(self, "_h", None) and _lib is not None:
            _lib.pccl_program_free(self._h)
            self._h = None

    def info(self) -> dict:
        out = ProgramInfo()
        check(lib().pccl_program_get_info(self._h, ctypes.byref(out)))
        return out.as_dict()

    def column_plan(self, staged: bool = False) -> dict:
        """Segments, instruction words and first-touch lists of the column plan (in place, or of a
        staged call that runs on the caller's tensors), plus the staged windows per rank."""
        L = lib()
        ns, ni, npre = ctypes.c_int(), ctypes.c_int(), ctypes.c_int()
        which = 1 if staged else 0
        check(L.pccl_program_get_column(self._h, which, None, 0, ctypes.byref(ns), None, 0, ctypes.byref(ni),
                                        None, 0, ctypes.byref(npre), None, None))
        R = self.info()["num_vranks"]
        segs = (ColumnSegment * max(ns.value, 1))()
        instrs = (ctypes.c_uint64 * max(ni.value, 1))()
        pre = (ctypes.c_uint64 * max(npre.value, 1))()
        win_in, win_out = (ctypes.c_int64 * (2 * R))(), (ctypes.c_int64 * (2 * R))()
        check(L.pccl_program_get_column(self._h, which, segs, ns.value, ctypes.byref(ns), instrs, ni.value,
                                        ctypes.byref(ni), pre, npre.value, ctypes.byref(npre), win_in, win_out))
        return {"segments": [segs[i] for i in range(ns.value)], "instrs": list(instrs)[:ni.value],
                "pre": list(pre)[:npre.value],
                "in_window": [(win_in[2 * r], win_in[2 * r + 1]) for r in range(R)],
                "out_window": [(win_out[2 * r], win_out[2 * r + 1]) for r in range(R)]}

    def ops(self):
        n = self.info()["num_data_ops"]
        arr = (LinkedOp * max(n, 1))()
        check(lib().pccl_program_get_ops(self._h, arr, n))
        return [arr[i] for i in range(n)]
