"""Engine facade: the reference's ``pccl.engine`` call surface over the HIP executor.

Reference (pccl/engine.py:11-71): ``register_operation(name, filename) -> bool``,
``execute_operation(name, input, output=None) -> Tensor`` (allocates ``empty_like`` and
synchronises), ``execute_operation_async`` (no sync), ``sync_operation(name)``,
``reset_signals(name)``, ``get_engine()``.  There every process is one rank and ``RANK`` comes from
the environment.  Here one process holds all R ranks of a schedule as *virtual ranks* on one GPU:

* collective form: ``engine.execute_operation(name, [in_0 .. in_{R-1}], [out_0 ..])`` — lists (or an
  ``[R, N]`` tensor) instead of one tensor;
* per-rank form, for code written against the reference: ``engine.rank(r)`` returns a view with the
  reference's exact single-rank signatures; ``execute_operation_async`` posts that rank's tensors and
  the launch happens when the last rank has posted (``execute_operation`` on a view is only legal
  once every other rank has posted, because it synchronises).

All work is enqueued on the current PyTorch stream, like the reference
(csrc/plugins/cuda/cuda_device.cc:245-248,301).
"""
from __future__ import annotations

import ctypes
import os
from typing import Dict, List, Optional, Sequence, Union

import torch

from . import _lib
from ._lib import PcclError

TensorList = Union[Sequence[torch.Tensor], torch.Tensor]


def _current_stream_ptr(device: torch.device) -> int:
    return torch.cuda.current_stream(device).cuda_stream


class Engine:
    def __init__(self, num_vranks: Optional[int] = None, device: int = 0):
        if num_vranks is None:
            num_vranks = int(os.environ.get("PCCL_VRANKS", "0"))
        if num_vranks <= 0:
            raise RuntimeError("number of virtual ranks not given: pass num_vranks or set PCCL_VRANKS")
        if not torch.cuda.is_available():
            raise RuntimeError("no GPU visible: the HIP executor has no CPU fallback")
        self.num_vranks = num_vranks
        self.device = torch.device("cuda", device)
        self._L = _lib.lib()
        h = ctypes.c_void_p()
        _lib.check(self._L.pccl_hip_create(ctypes.byref(h), device, num_vranks))
        self._h = h
        self._posted: Dict[str, Dict[int, tuple]] = {}
        self._elem_bytes: Dict[str, int] = {}      # per operation: element size of the graph's dtype
        self._views = [RankView(self, r) for r in range(num_vranks)]

    def close(self) -> None:
        if getattr(self, "_h", None):
            self._L.pccl_hip_destroy(self._h)
            self._h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    # -- registration -------------------------------------------------------------------------
    def register_operation(self, name: str, filename: str, rank: Optional[int] = None) -> bool:
        """Register rank ``rank``'s graph file; with ``rank=None`` ``filename`` must contain
        ``{rank}`` and all virtual ranks are registered.  Returns False when a file cannot be
        loaded (like the reference's ``regOp``); a bad primitive or dtype raises."""
        self._elem_bytes.pop(name, None)
        ranks = [rank] if rank is not None else list(range(self.num_vranks))
        if rank is None and "{rank}" not in filename:
            raise ValueError("register_operation without rank needs a '{rank}' placeholder in filename")
        for r in ranks:
            path = filename.format(rank=r) if "{rank}" in filename else filename
            rc = self._L.pccl_hip_register_file(self._h, name.encode(), r, path.encode())
            if rc in (_lib.ERR_NOT_FOUND, _lib.ERR_NOT_A_GRAPH):   # where the reference's loader returns false
                return False
            _lib.check(rc)
            if name not in self._elem_bytes:
                self._note_dtype(name, _lib.HostGraph.from_file(path))
        return True

    def register_operation_json(self, name: str, text: str, rank: int) -> bool:
        self._elem_bytes.pop(name, None)
        data = text.encode()
        _lib.check(self._L.pccl_hip_register_json(self._h, name.encode(), rank, data, len(data)))
        self._note_dtype(name, _lib.HostGraph.from_json(text))
        return True

    def _note_dtype(self, name: str, graph) -> None:
        """Remember the element size of the operation's graphs at registration (a host-side parse), so
        that checking the tensors of a call never has to link the operation: linking allocates, which
        a caller that is capturing its stream cannot have."""
        self._elem_bytes[name] = self._DTYPE_BYTES[graph.dtype]

    def last_error(self) -> str:
        return self._L.pccl_hip_last_error().decode(errors="replace")

    def set_option(self, key: str, value) -> None:
        """Option `key` (see pccl_hip_set_option in include/pccl_hip.h) takes text or a whole number;
        True and False are passed as 1 and 0."""
        if isinstance(value, bool):
            value = int(value)
        _lib.check(self._L.pccl_hip_set_option(self._h, key.encode(), str(value).encode()))

    def get_option(self, key: str) -> str:
        buf = ctypes.create_string_buffer(65536 if key == "signals" else 64)
        _lib.check(self._L.pccl_hip_get_option(self._h, key.encode(), buf, len(buf)))
        return buf.value.decode()

    # -- execution ----------------------------------------------------------------------------
    def _as_list(self, t: TensorList, what: str) -> List[torch.Tensor]:
        ts = list(t.unbind(0)) if isinstance(t, torch.Tensor) else list(t)
        if len(ts) != self.num_vranks:
            raise ValueError(f"{what}: expected {self.num_vranks} tensors, got {len(ts)}")
        for x in ts:
            if not x.is_cuda:
                raise ValueError(f"{what}: tensors must live on the GPU")
            if x.device != self.device:
                raise ValueError(f"{what}: tensor on {x.device}, the engine runs on {self.device}")
            if not x.is_contiguous():
                raise ValueError(f"{what}: tensors must be contiguous")
        return ts

    _DTYPE_BYTES = {0: 4, 1: 2, 2: 2, 3: 1, 4: 1, 5: 4}    # pccl_dtype -> bytes per element

    def _check_dtype(self, name: str, ts: List[torch.Tensor], what: str) -> None:
        """The library sees bytes, and the reference checks nothing (engine_c.cc:304-320): a tensor
        whose elements are not the size of the graph's dtype is certainly a mistake, so say so."""
        es = self._elem_bytes.get(name)
        if es is None:
            es = self._elem_bytes[name] = self._DTYPE_BYTES[self.op_info(name)["dtype"]]
        for x in ts:
            if x.element_size() != es:
                raise ValueError(f"{what}: {x.dtype} has {x.element_size()}-byte elements, "
                                 f"operation '{name}' was compiled for {es}-byte elements")

    def _ptrs(self, ts: List[torch.Tensor]):
        return (ctypes.c_void_p * len(ts))(*[x.data_ptr() for x in ts])

    def _launch(self, name: str, inputs: List[torch.Tensor], outputs: List[torch.Tensor], sync: bool):
        nb_in, nb_out = inputs[0].nbytes, outputs[0].nbytes
        if any(x.nbytes != nb_in for x in inputs) or any(x.nbytes != nb_out for x in outputs):
            raise ValueError("all ranks must pass tensors of the same size")
        self._check_dtype(name, inputs, "inputs")
        self._check_dtype(name, outputs, "outputs")
        _lib.check(self._L.pccl_hip_execute(self._h, name.encode(), self._ptrs(inputs), self._ptrs(outputs),
                                            nb_in, nb_out, _current_stream_ptr(self.device), int(sync)))

    def execute_operation(self, name: str, inputs: TensorList, outputs: Optional[TensorList] = None):
        ins = self._as_list(inputs, "inputs")
        outs = [torch.empty_like(x) for x in ins] if outputs is None else self._as_list(outputs, "outputs")
        self._launch(name, ins, outs, True)
        return outs

    def execute_operation_async(self, name: str, inputs: TensorList, outputs: Optional[TensorList] = None):
        ins = self._as_list(inputs, "inputs")
        outs = [torch.empty_like(x) for x in ins] if outputs is None else self._as_list(outputs, "outputs")
        self._launch(name, ins, outs, False)
        return outs

    def execute_inplace(self, name: str, bufs: TensorList, sync: bool = False):
        """Zero-copy execution: ``bufs[r]`` is rank ``r``'s buffer and is updated in place."""
        bs = self._as_list(bufs, "bufs")
        self._check_dtype(name, bs, "bufs")
        # the library checks the program's extent against one size: the smallest buffer's
        _lib.check(self._L.pccl_hip_execute_inplace(self._h, name.encode(), self._ptrs(bs), min(b.nbytes for b in bs),
                                                    _current_stream_ptr(self.device), int(sync)))
        return bs

    def execute_inplace_static(self, name: str, bufs: TensorList, sync: bool = False):
        """``execute_inplace`` for callers that cannot allocate: one launch of the persistent runner in
        the GPU's static workspace (see ``pccl_hip_execute_inplace_static``).  No counterpart in the
        reference."""
        bs = self._as_list(bufs, "bufs")
        self._check_dtype(name, bs, "bufs")
        _lib.check(self._L.pccl_hip_execute_inplace_static(self._h, name.encode(), self._ptrs(bs), min(b.nbytes for b in bs),
                                                           _current_stream_ptr(self.device), int(sync)))
        return bs

    def prepare(self, name: str, inputs: TensorList, outputs: Optional[TensorList] = None) -> "PreparedCall":
        """Check the tensors and build the argument arrays once; the returned object launches the
        operation on those tensors with nothing but the C call per invocation (for loops that issue
        the same small collective over and over: the checks and array building of
        ``execute_operation_async`` cost more than a small kernel takes).  ``outputs=None`` means
        in place on ``inputs``.  No counterpart in the reference."""
        ins = self._as_list(inputs, "inputs")
        outs = None if outputs is None else self._as_list(outputs, "outputs")
        if any(x.nbytes != ins[0].nbytes for x in ins) or (outs and any(x.nbytes != outs[0].nbytes for x in outs)):
            raise ValueError("all ranks must pass tensors of the same size")
        self._check_dtype(name, ins, "inputs")
        if outs:
            self._check_dtype(name, outs, "outputs")
        return PreparedCall(self, name, ins, outs)

    def sync_operation(self, name: str) -> None:
        _lib.check(self._L.pccl_hip_sync(self._h, name.encode()))

    def reset_signals(self, name: str) -> None:
        """Zero every counting semaphore of the engine (reference ``Engine::resetSignals``,
        ``csrc/engine_c.cc:576-593``: the signal region is one per engine, whichever operation is named)."""
        _lib.check(self._L.pccl_hip_reset_signals(self._h, name.encode()))

    def signals(self) -> dict:
        """The semaphores that executions so far have left above zero: ``{(rank, signal_id): count}``.
        The next execution of any operation finds them (a wait passes on a count above zero and takes
        one, reference ``csrc/plugins/cuda/cuda_executor.cu:425-445``)."""
        out = {}
        for item in filter(None, self.get_option("signals").split(",")):
            key, _, count = item.partition("=")
            rank, _, sid = key.partition(":")
            out[(int(rank), int(sid))] = int(count)
        return out

    def op_info(self, name: str) -> dict:
        out = _lib.ProgramInfo()
        _lib.check(self._L.pccl_hip_op_info(self._h, name.encode(), ctypes.byref(out)))
        return out.as_dict()

    def last_kernel_ms(self, name: str) -> float:
        ms = ctypes.c_float()
        _lib.check(self._L.pccl_hip_last_kernel_ms(self._h, name.encode(), ctypes.byref(ms)))
        return ms.value

    # -- per-rank views -----------------------------------------------------------------------
    def rank(self, r: int) -> "RankView":
        return self._views[r]

    def _post(self, name: str, r: int, inp: torch.Tensor, out: torch.Tensor, sync: bool):
        slot = self._posted.setdefault(name, {})
        if r in slot:
            raise RuntimeError(f"rank {r} posted '{name}' twice before the other ranks arrived")
        slot[r] = (inp, out)
        if len(slot) < self.num_vranks:
            if sync:
                del slot[r]
                raise RuntimeError(
                    f"execute_operation('{name}') on rank {r} would block: only {len(slot) + 1} of "
                    f"{self.num_vranks} virtual ranks have posted; post the others with "
                    "execute_operation_async first")
            return
        ins = self._as_list([slot[i][0] for i in range(self.num_vranks)], "inputs")
        outs = self._as_list([slot[i][1] for i in range(self.num_vranks)], "outputs")
        del self._posted[name]
        self._launch(name, ins, outs, sync)


class PreparedCall:
    """An operation bound to fixed tensors (see ``Engine.prepare``).  Keeps the tensors alive."""

    def __init__(self, engine: Engine, name: str, inputs: List[torch.Tensor], outputs: Optional[List[torch.Tensor]]):
        self._engine, self._name = engine, name.encode()
        self.inputs, self.outputs = inputs, outputs if outputs is not None else inputs
        self._in = engine._ptrs(inputs)
        self._out = None if outputs is None else engine._ptrs(outputs)
        self._nb_in = inputs[0].nbytes
        self._nb_out = self.outputs[0].nbytes
        self._execute, self._inplace = engine._L.pccl_hip_execute, engine._L.pccl_hip_execute_inplace

    def __call__(self, sync: bool = False, stream: Optional[int] = None):
        """Launch on `stream` (a raw stream handle) or on the current torch stream."""
        e = self._engine
        st = _current_stream_ptr(e.device) if stream is None else stream
        if self._out is None:
            rc = self._inplace(e._h, self._name, self._in, self._nb_in, st, int(sync))
        else:
            rc = self._execute(e._h, self._name, self._in, self._out, self._nb_in, self._nb_out, st, int(sync))
        if rc < 0:
            _lib.check(rc)
        return self.outputs


class RankView:
    """The reference's single-rank API for one virtual rank."""

    def __init__(self, engine: Engine, rank: int):
        self.engine, self.rank = engine, rank

    def register_operation(self, name: str, filename: str) -> bool:
        return self.engine.register_operation(name, filename, rank=self.rank)

    def execute_operation(self, name, input_tensor, output_tensor=None):
        if output_tensor is None:
            output_tensor = torch.empty_like(input_tensor)
        self.engine._post(name, self.rank, input_tensor, output_tensor, True)
        return output_tensor

    def execute_operation_async(self, name, input_tensor, output_tensor=None):
        if output_tensor is None:
            output_tensor = torch.empty_like(input_tensor)
        self.engine._post(name, self.rank, input_tensor, output_tensor, False)
        return output_tensor

    def sync_operation(self, name):
        self.engine.sync_operation(name)

    def reset_signals(self, name):
        self.engine.reset_signals(name)


_engine_instance: Optional[Engine] = None


def initialize_engine(num_vranks: Optional[int] = None, device: int = 0) -> Engine:
    """Create the process-wide engine (the reference's ``initialize_engine(group)`` exchanges
    endpoints between processes; with virtual ranks there is nothing to exchange)."""
    global _engine_instance
    if _engine_instance is not None:
        _engine_instance.close()
    _engine_instance = Engine(num_vranks, device)
    return _engine_instance


def get_engine() -> Engine:
    global _engine_instance
    if _engine_instance is None:
        _engine_instance = Engine()
    return _engine_instance


def register_operation(name, filename, rank=None):
    return get_engine().register_operation(name, filename, rank)


def execute_operation(name, input_tensor, output_tensor=None):
    return get_engine().execute_operation(name, input_tensor, output_tensor)


def execute_operation_async(name, input_tensor, output_tensor=None):
    return get_engine().execute_operation_async(name, input_tensor, output_tensor)


def sync_operation(name):
    return get_engine().sync_operation(name)


def reset_signals(name):
    return get_engine().reset_signals(name)
