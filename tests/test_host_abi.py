"""Host-side behaviour of the C ABI (no GPU): the library loads and exports what the header
declares, graphs load with the reference's field mapping and error behaviour, fused steps group
like the reference's descriptor builder, and the cross-rank linker finds deadlocks and races.
"""
import ctypes
import json
import os
import re

import pytest

from helpers import ROOT, graph_jsons, oracle
from pccl_amd import _lib
from pccl_amd._lib import (ERR_INVALID, ERR_LINK, ERR_NOT_A_GRAPH, ERR_NOT_FOUND, ERR_PARSE, ERR_UNSUPPORTED, HostGraph,
                           HostProgram, PcclError)
from pccl_amd.dsl import CommunicationOp, compile_to_json_string


def test_library_exports_every_declared_symbol():
    header = open(os.path.join(ROOT, "include", "pccl_hip.h")).read()
    declared = set(re.findall(r"\b(pccl_(?:hip|graph|program)_\w+)\s*\(", header))
    assert len(declared) >= 30
    L = _lib.lib()
    missing = [n for n in sorted(declared) if not hasattr(L, n)]
    assert not missing, missing
    assert declared == set(_lib.EXPORTS)
    assert b"gfx950" in L.pccl_hip_version()


def test_struct_layouts_match_the_reference():
    """sizes / offsets of the reference structs (proxy_trigger.h:8-16, primitive.h:8-17, fused_step.h:7-22)."""
    assert ctypes.sizeof(_lib.Trigger) == 32
    assert [getattr(_lib.Trigger, f).offset for f in ("primitive_type", "op_index", "peer_rank", "offset_0",
                                                      "offset_1", "offset_2", "size")] == [0, 4, 8, 12, 16, 20, 24]
    assert ctypes.sizeof(_lib.PrimitiveMeta) == 88
    assert ctypes.sizeof(_lib.FusedStep) == 44


def test_no_device_means_error_not_fallback():
    import torch
    if torch.cuda.is_available():
        pytest.skip("a GPU is present")
    h = ctypes.c_void_p()
    rc = _lib.lib().pccl_hip_create(ctypes.byref(h), 0, 8)
    assert rc == _lib.ERR_HIP
    assert b"no CPU fallback" in _lib.lib().pccl_hip_last_error()
    from pccl_amd.engine import Engine
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        Engine(8, 0)


# ------------------------------------------------------------------------------- graph loading

def test_trigger_fields_agree_with_an_independent_parse():
    """The product's C++ loader against the oracle's Python loader (both follow sm_channel.h /
    tma_channel.h) on every golden graph."""
    idx = json.load(open(os.path.join(ROOT, "tests/golden/graphs/index.json")))
    kinds = {1: "reduce", 2: "copy", 3: "notify", 4: "wait"}
    for case in idx:
        for rank in range(case["world_size"]):
            path = os.path.join(ROOT, "tests/golden/graphs", f"{case['stem']}_rank{rank}.json")
            g = HostGraph.from_file(path)
            o = oracle.Graph.from_file(path)
            trig, n = g.triggers()
            meta, _ = g.meta()
            assert n == o.n and g.collective_type == o.collective_type
            assert g.dtype == o.dtype and g.tensor_elems == case["tensor_size"]
            for i in range(n):
                t, m, q = trig[i], meta[i], o.table[i]
                assert (t.op_index, t.peer_rank, m.channel, m.num_dependencies, m.num_next_ops) == \
                       (q.index, q.peer, q.channel, q.ndeps, q.nnext)
                pt = t.primitive_type
                if kinds[q.kind] == "reduce":
                    assert pt in (1 + o.dtype, 33 + o.dtype)
                    assert (t.offset_0, t.offset_1, t.offset_2, t.size) == (q.off0, q.off1, q.off2, q.size)
                elif kinds[q.kind] == "copy":
                    assert pt in (6 + o.dtype, 28 + o.dtype)
                    assert (t.offset_0, t.offset_1, t.size) == (q.off0, q.off1, q.size)
                else:
                    assert pt == (22 if kinds[q.kind] == "notify" else 21) and t.offset_0 == q.off0
                assert list(m.next_primitive_index)[:m.num_next_ops] == list(q.next)[:q.nnext]


def test_primitive_ids_distinguish_sm_and_tma():
    sm = HostGraph.from_json(graph_jsons("ring", "build_allreduce", 2, 2048, "bfloat16", "sm")[0]).triggers()[0]
    tma = HostGraph.from_json(graph_jsons("ring", "build_allreduce", 2, 2048, "bfloat16", "tma")[0]).triggers()[0]
    assert sm[2].primitive_type == 3 and sm[5].primitive_type == 8        # cuda_reduce_bf16, cuda_copy_bf16
    assert tma[2].primitive_type == 35 and tma[5].primitive_type == 30    # cuda_tma_reduce_bf16, cuda_tma_copy_bf16


def _doc(**over):
    doc = json.loads(graph_jsons("ring", "build_allreduce", 2, 2048, "float32", "sm")[0])
    doc.update(over)
    return doc


def _load_err(doc_or_text):
    text = doc_or_text if isinstance(doc_or_text, str) else json.dumps(doc_or_text)
    with pytest.raises(PcclError) as e:
        HostGraph.from_json(text)
    return e.value


def test_load_errors():
    with pytest.raises(PcclError) as e:
        HostGraph.from_file("/nonexistent/graph.json")
    assert e.value.code == ERR_NOT_FOUND                       # reference: regOp returns false
    d = _doc(); del d["operations"]
    assert _load_err(d).code == ERR_NOT_A_GRAPH                 # reference: returns false
    d = _doc(); del d["operations"][3]["primitive"]
    assert "index/executor/primitive" in str(_load_err(d)) and _load_err(d).code == ERR_NOT_A_GRAPH   # false there too
    d = _doc(); d["operations"][2]["primitive"] = "sm.scatter"
    assert "unknown primitive" in str(_load_err(d))             # reference: throws
    d = _doc(); d["tensor_info"]["dtype"] = "float64"
    assert "Unsupported dtype" in str(_load_err(d))             # reference: throws (sm_channel.h:71)
    d = _doc(); d["tensor_info"]["dtype"] = "float8_e4m3"
    assert HostGraph.from_json(json.dumps(d)).dtype == 3              # fp8 graphs load (reference vec.h:272-426)
    d = _doc(); d["operations"][2]["executor"] = "cuda_ce"
    assert _load_err(d).code == ERR_UNSUPPORTED
    d = _doc(); d["operations"][2]["params"]["reduce_op"] = "avg"
    assert _load_err(d).code == ERR_UNSUPPORTED
    d = _doc(); del d["operations"][2]["params"]["count"]
    assert "params.count" in str(_load_err(d))
    d = _doc(); d["operations"][0]["params"]["signal_id"] = 4096
    assert "signal_id" in str(_load_err(d))
    d = _doc(); d["operations"][1]["dependencies"] = [99]
    assert "unknown operation index" in str(_load_err(d))
    assert _load_err("{not json").code == ERR_PARSE
    assert _load_err('{"operations": [1, 2').code == ERR_PARSE


def test_int32_and_max_are_accepted_as_extensions():
    g = HostGraph.from_json(graph_jsons("tree", "build_allreduce", 4, 1024, "int32", "sm", reduce_op="max")[0])
    trig, n = g.triggers()
    red = [trig[i] for i in range(n) if trig[i].primitive_type == 64]
    assert red and all(t.redop == 1 for t in red)
    assert g.dtype == 5


def test_graph_from_triggers_round_trip():
    text = graph_jsons("ring", "build_allreduce", 4, 4096, "float16", "tma", 2)[1]
    g = HostGraph.from_json(text)
    trig, n = g.triggers()
    meta, _ = g.meta()
    g2 = HostGraph.from_triggers(trig, meta, g.collective_type)
    t2, n2 = g2.triggers()
    assert n2 == n and g2.dtype == g.dtype and g2.collective_type == "allreduce"
    for i in range(n):
        assert bytes(trig[i])[:28] == bytes(t2[i])[:28]


def test_trigger_arrays_are_range_checked_like_documents():
    """The trigger path (what a DevicePlugin adapter hands over) refuses what the JSON path refuses:
    negative offsets and sizes, ranges past 2^31 - 1 elements, signal ids outside the signal array.
    Host only: such a graph must never reach a kernel."""
    text = graph_jsons("ring", "build_allreduce", 2, 2048, "float32", "sm", 1)[0]
    g = HostGraph.from_json(text)
    meta, _ = g.meta()

    def damaged(pick, **fields):
        trig, n = g.triggers()
        i = next(k for k in range(n) if pick(trig[k]))
        for name, value in fields.items():
            setattr(trig[i], name, value)
        with pytest.raises(PcclError) as e:
            HostGraph.from_triggers(trig, meta, "allreduce")
        assert e.value.code == ERR_PARSE, str(e.value)
        return str(e.value)

    is_copy = lambda t: t.primitive_type == 6
    is_reduce = lambda t: t.primitive_type == 1
    is_signal = lambda t: t.primitive_type in (21, 22)
    assert "negative" in damaged(is_copy, offset_1=-100000, size=1024)
    assert "negative" in damaged(is_copy, offset_0=-1)
    assert "negative" in damaged(is_copy, size=-5)
    assert "negative" in damaged(is_reduce, offset_2=-16)
    assert "32-bit element range" in damaged(is_copy, offset_1=2**31 - 1000, size=1024)
    assert "32-bit element range" in damaged(is_reduce, offset_2=2**31 - 1, size=2)
    assert "signal_id" in damaged(is_signal, offset_0=4096)
    assert "signal_id" in damaged(is_signal, offset_0=-1)
    # untouched arrays still load, and a copy's unused third offset is ignored
    trig, n = g.triggers()
    i = next(k for k in range(n) if is_copy(trig[k]))
    trig[i].offset_2 = -7
    assert HostGraph.from_triggers(trig, meta, "allreduce").num_ops == n


# ------------------------------------------------------------------------------- fused steps

def test_fused_steps_two_rank_ring():
    """The worked example: notify/wait/data grouping of reference graph_builder.cc:236-311."""
    g = HostGraph.from_file(os.path.join(ROOT, "tests/golden/graphs/ring_ar_sm_w2_n2048_bf16_c1_rank0.json"))
    steps, offs = g.fused_steps()
    assert offs == [0, 3]
    s0, s1, s2 = steps
    assert (s0.has_notify, s0.notify_peer_rank, s0.notify_signal_id, s0.has_wait, s0.wait_signal_id) == (1, 1, 100, 1, 100)
    assert (s0.primitive_type, s0.peer_rank, s0.offset_0, s0.offset_1, s0.offset_2, s0.size) == (3, 1, 1024, 1024, 1024, 1024)
    assert (s1.has_notify, s1.notify_signal_id, s1.has_wait, s1.primitive_type, s1.offset_0, s1.size) == (1, 0, 1, 8, 0, 1024)
    assert (s2.has_notify, s2.has_wait, s2.primitive_type) == (1, 1, 0)


def test_fused_steps_counts():
    g = HostGraph.from_json(graph_jsons("ring", "build_allreduce", 8, 8192 * 4, "bfloat16", "sm", 4)[0])
    steps, offs = g.fused_steps()
    assert offs == [0, 15, 30, 45, 60]                       # 7 reduce + 7 copy + 1 signal-only per channel
    assert sum(1 for s in steps if 1 <= s.primitive_type <= 5) == 28
    g = HostGraph.from_json(graph_jsons("rhd", "build_allreduce", 16, 4096, "float32", "sm")[3])
    assert len(g.fused_steps()[0]) == 9


def test_fused_steps_fall_back_like_the_reference():
    # alltoall: a data op directly follows a data op -> not a fused chain
    g = HostGraph.from_json(graph_jsons("ring", "build_alltoall", 4, 4096, "bfloat16")[0])
    with pytest.raises(PcclError) as e:
        g.fused_steps()
    assert e.value.code == ERR_UNSUPPORTED
    # ring with 32 ranks and 4 channels needs 252 > 128 steps
    g = HostGraph.from_json(graph_jsons("ring", "build_allreduce", 32, 4096 * 32, "bfloat16", "sm", 4)[0])
    with pytest.raises(PcclError):
        g.fused_steps()


# ------------------------------------------------------------------------------- linker

def _link(jsons):
    return HostProgram([HostGraph.from_json(j) for j in jsons])


def test_element_counts_are_32_bit_like_the_reference_descriptors():
    """Offsets and sizes are ints in the reference's trigger and fused step (include/engine/fused_step.h:11-14,
    cuda_executor.cu:63-72): a graph whose op reaches 2^31 elements is refused at load time, one that
    stays a single element below loads, links and keeps its descriptor forms exact."""
    n = (1 << 31) - 2
    jsons = graph_jsons("ring", "build_allreduce", 2, n, "float32", "sm", 1)
    g = HostGraph.from_json(jsons[0])
    trig, cnt = g.triggers()
    assert max(trig[i].offset_0 + trig[i].size for i in range(cnt) if trig[i].primitive_type in (1, 3, 64, 65, 8)) <= n
    assert any(trig[i].offset_0 == n // 2 and trig[i].size == n // 2 for i in range(cnt))
    assert _link(jsons).info()["algorithmic_bytes"] == 5 * n * 4
    with pytest.raises(PcclError) as e:
        HostGraph.from_json(graph_jsons("ring", "build_allreduce", 2, 1 << 32, "float32", "sm", 1)[0])
    assert e.value.code == ERR_PARSE and "32-bit element range" in str(e.value)


def test_log_level_switch():
    """PCCL_LOG_LEVEL as in the reference (csrc/common/logging.cc:6-35): nothing below WARN by default;
    INFO repeats the message of a failing call on stderr, stdout stays untouched."""
    import subprocess
    import sys
    code = ("import sys; sys.path.insert(0, %r); from pccl_amd._lib import HostGraph, PcclError\n"
            "try: HostGraph.from_json('{}')\n"
            "except PcclError as e: print('code', e.code)\n") % ROOT
    for level, expect in ((None, False), ("INFO", True), ("ERROR", False), ("nonsense", False)):
        env = {k: v for k, v in os.environ.items() if k != "PCCL_LOG_LEVEL"}
        if level:
            env["PCCL_LOG_LEVEL"] = level
        out = subprocess.run([sys.executable, "-c", code], env=env, capture_output=True, text=True, timeout=120)
        assert out.stdout.strip() == f"code {ERR_NOT_A_GRAPH}"
        assert ("[pccl] [info] call failed (-7)" in out.stderr) == expect, (level, out.stderr)


def test_program_info_closed_forms():
    world, n = 8, 8192 * 4
    info = _link(graph_jsons("ring", "build_allreduce", world, n, "bfloat16", "sm", 4)).info()
    S = n * 2
    assert info["num_data_ops"] == 448 and info["num_ops"] == 8 * 176
    assert info["num_levels"] == 2 * (world - 1)
    assert info["algorithmic_bytes"] == 5 * (world - 1) * S
    assert info["position_aligned"] == 1 and info["num_segments"] == 32
    # column plan: every rank buffer read once and written once
    assert info["column_load_bytes"] == world * S and info["column_store_bytes"] == world * S
    assert info["residual_signals"] == 0 and info["buffer_elems"] == n
    info = _link(graph_jsons("rhd", "build_allreduce", 16, 4096, "float32", "sm")).info()
    assert info["num_levels"] == 8 and info["algorithmic_bytes"] == 5 * 15 * 4096 * 4
    info = _link(graph_jsons("tree", "build_allreduce", 32, 4096, "float32", "sm")).info()
    assert info["num_levels"] == 10 and info["num_data_ops"] == 62
    # ragged pieces of one schedule step touch disjoint ranges: they share a level
    from pccl_amd.dsl import ragged_cuts
    info = _link(graph_jsons("tree", "build_allreduce", 32, 4099, "int32", "sm", cuts=ragged_cuts(4099, 8))).info()
    assert info["num_levels"] == 10 and info["num_data_ops"] == 62 * 8
    info = _link(graph_jsons("ring", "build_alltoall", 4, 4096, "bfloat16")).info()
    assert info["position_aligned"] == 0 and info["buffer_elems"] == 2 * 4096


def test_linked_dependencies_of_the_ring():
    world, n = 4, 4096
    ops = _link(graph_jsons("ring", "build_allreduce", world, n, "float32", "sm")).ops()
    by = {(o.rank, o.level): (k, o) for k, o in enumerate(ops)}
    for (rank, level), (k, o) in by.items():
        deps = sorted(list(o.deps)[:o.num_deps])
        if level == 0:
            assert deps == []
        else:   # the producer of the chunk this op pulls: the previous rank's previous op.  (The own
                # previous op works on another chunk: chain order, but no memory conflict.)
            assert by[((rank - 1) % world, level - 1)][0] in deps
            assert all(ops[d].level < level for d in deps)
        assert o.peer_rank == (rank - 1) % world
        assert o.is_reduce == (1 if level < world - 1 else 0)


def _two_rank(build):
    out = []
    for rank in range(2):
        with CommunicationOp(name=f"g{rank}") as op:
            op.tensor(dtype="float32", shape=(64,))
            build(op, rank, 1 - rank)
        out.append(compile_to_json_string(op.get_graph()))
    return out


def _link_err(jsons):
    with pytest.raises(PcclError) as e:
        _link(jsons)
    assert e.value.code == ERR_LINK
    return str(e.value)


def test_linker_reports_deadlock():
    msg = _link_err(_two_rank(lambda op, me, other: (op.wait_notify(signal_id=3, source_rank=other),
                                                     op.sm_copy(source_rank=other, src_offset=0, dst_offset=0, size=64))))
    assert "deadlock" in msg and "signal 3" in msg


def test_linker_reports_unordered_conflicting_accesses():
    # both ranks copy from the other into the range the other is reading, with no ordering at all
    msg = _link_err(_two_rank(lambda op, me, other: op.sm_copy(source_rank=other, src_offset=0, dst_offset=0, size=64)))
    assert "data race" in msg
    # the same exchange made safe: disjoint halves
    jsons = _two_rank(lambda op, me, other: op.sm_copy(source_rank=other, src_offset=32 * other, dst_offset=32 * other, size=32))
    assert _link(jsons).info()["num_data_ops"] == 2


def test_linker_rejects_bad_ranks_and_mixed_types():
    msg = _link_err(_two_rank(lambda op, me, other: op.sm_copy(source_rank=5, src_offset=0, dst_offset=0, size=8)))
    assert "names rank 5" in msg
    a = graph_jsons("ring", "build_allreduce", 2, 2048, "float32", "sm")
    b = graph_jsons("ring", "build_allreduce", 2, 2048, "bfloat16", "sm")
    assert "dtype" in _link_err([a[0], b[1]])
    c = graph_jsons("ring", "build_reduce_scatter", 2, 2048, "float32", "sm")
    assert "collective_type" in _link_err([a[0], c[1]])


def test_linker_rejects_partially_overlapping_in_place_op():
    msg = _link_err(_two_rank(lambda op, me, other: op.sm_reduce(source_rank=other, src_offset=0, dst_offset=8,
                                                                 remote_offset=0, count=32) if me == 0 else
                              op.notify(signal_id=1, target_rank=other)))
    assert "overlap" in msg


def test_residual_signals_are_counted():
    jsons = _two_rank(lambda op, me, other: op.notify(signal_id=9, target_rank=other))   # never awaited
    info = _link(jsons).info()
    assert info["residual_signals"] == 2
    assert info["race_checked"] == 1 and info["order_checked"] == 1


def test_linking_for_counts_that_earlier_executions_left():
    """The linker given the semaphore state an execution finds (reference: one signal region per
    engine, cleared only by resetSignals, csrc/engine_c.cc:576-593; a wait passes on a count above
    zero and takes one, cuda_executor.cu:425-445) against the oracle given the same state: the same
    programs run or deadlock, and counts move by notifies - waits."""
    import json
    import numpy as np
    from helpers import carry_ops, oracle
    n = 64
    jsons = carry_ops(n)
    hg = {k: [HostGraph.from_json(j) for j in v] for k, v in jsons.items()}
    og = {k: [oracle.Graph(json.loads(j)) for j in v] for k, v in jsons.items()}
    uses = {k: HostProgram(v, {(1, 5): 1} if k == "take" else None).signals() for k, v in hg.items()}
    assert uses == {"give": {(1, 5): (2, 1)}, "take": {(1, 5): (0, 1)}, "pair": {(1, 5): (1, 1)}}
    for count in range(0, 4):
        for name in ("give", "take", "pair"):
            carried = {(1, 5): count} if count else {}
            sig = oracle.new_signals(2)
            sig[1, 5] = count
            bufs = [np.zeros(n, dtype=np.float32) for _ in range(2)]
            try:
                oracle.run(og[name], bufs, signals=sig)
                oracle_runs = True
            except oracle.OracleError as e:
                assert "deadlock" in str(e)
                oracle_runs = False
            try:
                prog = HostProgram(hg[name], carried)
                links, msg = True, ""
            except PcclError as e:
                links, msg = False, str(e)
            if name == "pair" and count > 0:
                # the oracle runs it in one of the orders the semaphores allow; the linker sees that the
                # copy is no longer ordered after the reduce it reads from
                assert oracle_runs and not links and "data race" in msg
                continue
            assert links == oracle_runs, (name, count, msg)
            if links:
                notifies, waits = prog.signals()[(1, 5)]
                assert int(sig[1, 5]) == count + notifies - waits
                assert prog.info()["residual_signals"] == (0 if notifies == waits else 1)
            else:
                assert "deadlock" in msg and "signal 5" in msg
    # a count on another semaphore, or on the same id of the other rank, changes nothing
    assert "deadlock" in _link_err_carried(hg["take"], {(0, 5): 3, (1, 6): 2})
    # the two leftover waits of two ranks are told apart: one count lets one wait through
    both = _two_rank(lambda op, me, other: (op.wait_notify(signal_id=2, source_rank=other),
                                            op.sm_copy(source_rank=other, src_offset=32 * other, dst_offset=32 * other, size=32)))
    hb = [HostGraph.from_json(j) for j in both]
    assert "rank 1" in _link_err_carried(hb, {(0, 2): 1})
    assert HostProgram(hb, {(0, 2): 1, (1, 2): 4}).info()["num_data_ops"] == 2


def _link_err_carried(graphs, carried):
    with pytest.raises(PcclError) as e:
        HostProgram(graphs, carried)
    assert e.value.code == ERR_LINK
    return str(e.value)


def test_linker_says_when_semaphores_do_not_balance():
    """A notify without a wait leaves its semaphore above zero, and the next execution of any
    operation finds it there (signals are only zeroed by resetSignals, csrc/engine_c.cc:576-593, and a
    wait passes on any count above zero, cuda_executor.cu:425-445): said at WARN level when the
    program is linked.  A balanced graph links silently.  A program too large for the ambiguity and
    race checks says that they were skipped."""
    import subprocess
    import sys
    code = ("import sys, json; sys.path.insert(0, %r); sys.path.insert(0, %r)\n"
            "from pccl_amd._lib import HostGraph, HostProgram\n"
            "from pccl_amd.dsl import CommunicationOp, compile_to_json_string\n"
            "from helpers import graph_jsons\n"
            "def rank(me, other, extra):\n"
            "    with CommunicationOp(name='r%%d' %% me) as op:\n"
            "        op.tensor(dtype='float32', shape=(64,))\n"
            "        op.notify(signal_id=1, target_rank=other); op.wait_notify(signal_id=1, source_rank=other)\n"
            "        op.sm_copy(source_rank=other, src_offset=me * 32, dst_offset=me * 32, size=32)\n"
            "        if extra: op.notify(signal_id=9, target_rank=other)\n"
            "        return compile_to_json_string(op.get_graph())\n"
            "which = sys.argv[1]\n"
            "if which == 'big': js = graph_jsons('ring', 'build_allreduce', 64, 64 * 4 * 4, 'float32', 'sm', 4)\n"
            "else: js = [rank(0, 1, which == 'unbalanced'), rank(1, 0, which == 'unbalanced')]\n"
            "info = HostProgram([HostGraph.from_json(j) for j in js]).info()\n"
            "print(info['residual_signals'], info['order_checked'], info['race_checked'])\n") % (ROOT, os.path.join(ROOT, "tests"))
    env = {k: v for k, v in os.environ.items() if k != "PCCL_LOG_LEVEL"}

    def run(which):
        out = subprocess.run([sys.executable, "-c", code, which], env=env, capture_output=True, text=True, timeout=300)
        assert out.returncode == 0, out.stderr
        return out.stdout.split(), out.stderr

    vals, err = run("unbalanced")
    assert vals == ["2", "1", "1"]
    assert "[pccl] [warning]" in err and "leaves 2 semaphore(s) at another count" in err and "carried into the next execution" in err
    vals, err = run("balanced")
    assert vals == ["0", "1", "1"] and "[pccl]" not in err
    vals, err = run("big")     # 64 ranks x 4 channels: more ops than the quadratic checks take
    assert vals[1:] == ["0", "0"]
    assert "[pccl] [warning]" in err and "too many for the notify/wait ambiguity check" in err


def test_reference_numbered_pipeline_schedule_is_reported_as_deadlock():
    """The pipelined ring of the reference's bandwidth script (tests/bench_allreduce_tma_bw.py:119-186)
    numbers waits and notifies with one running counter, so every wait after the first step is on
    an id nobody notifies.  The reference's wait has no bail-out (cuda_executor.cu:946-961 spins
    until the count is above zero), so it can only pass there on counts left over from earlier
    executions.  Linked with exact semaphore semantics, every count starting at zero, this is a
    deadlock, reported at link time, by the product's linker and by the oracle alike."""
    from helpers import pipelined_ring_allreduce, oracle_buffers, seeded_inputs
    from pccl_amd.dsl import compile_to_json_string
    world, n = 4, 4096
    jsons = [compile_to_json_string(pipelined_ring_allreduce(r, world, n, "float32", 2)) for r in range(world)]
    with pytest.raises(PcclError, match="deadlock"):
        HostProgram([HostGraph.from_json(j) for j in jsons])
    with pytest.raises(Exception, match="deadlock"):
        oracle_buffers(jsons, seeded_inputs("randn", world, n, "float32"), "float32")
    # the same schedule with paired signal ids links, race-free
    jsons = [compile_to_json_string(pipelined_ring_allreduce(r, world, n, "float32", 2, paired_signals=True))
             for r in range(world)]
    info = HostProgram([HostGraph.from_json(j) for j in jsons]).info()
    assert info["residual_signals"] == 0 and info["position_aligned"] == 1 and info["num_data_ops"] == 24


def test_alltoall_gather_plan():
    """A one-channel alltoall composes into R*R direct input-to-output copies; allreduce graphs and
    the two-channel alltoall (whose scratch chunks the engine's output rule reads are not all
    written by the program) have no such plan and are staged."""
    from helpers import graph_jsons
    for world in (3, 4, 8):
        jsons = graph_jsons("ring", "build_alltoall", world, world * 512, "bfloat16", "sm", 1)
        assert HostProgram([HostGraph.from_json(j) for j in jsons]).info()["num_gather_copies"] == world * world
    jsons = graph_jsons("ring", "build_alltoall", 4, 4096, "bfloat16", "sm", 2)
    assert HostProgram([HostGraph.from_json(j) for j in jsons]).info()["num_gather_copies"] == 0
    jsons = graph_jsons("ring", "build_allreduce", 4, 4096, "bfloat16", "sm", 1)
    assert HostProgram([HostGraph.from_json(j) for j in jsons]).info()["num_gather_copies"] == 0


def test_damaged_documents_are_errors_not_crashes():
    """Truncated, corrupted and out-of-range graph documents come back as error codes (or load, and
    then link or fail to link cleanly): nothing crosses the C ABI as a crash or an exception."""
    import random
    L = _lib.lib()
    rng = random.Random(7)
    stems = ["ring_ar_sm_w2_n2048_bf16_c1_rank0", "ring_ar_sm_w4_n4096_f32_c2_rank0", "tree_ar_sm_w8_n1024_f32_c1_rank0"]
    paths = [os.path.join(ROOT, "tests/golden/graphs", s + ".json") for s in stems]
    loaded = failed = 0
    for path in paths:
        text = open(path, "rb").read()
        for _ in range(150):
            b = bytearray(text)
            kind = rng.randrange(4)
            if kind == 0:
                b = b[:rng.randrange(len(b))]
            elif kind == 1:
                for _ in range(rng.randrange(1, 6)):
                    b[rng.randrange(len(b))] = rng.randrange(256)
            elif kind == 2:
                i = rng.randrange(len(b))
                del b[i:i + rng.randrange(1, 40)]
            else:
                s = b.decode("latin1")
                nums = list(re.finditer(r"\d+", s))
                m = rng.choice(nums)
                s = s[:m.start()] + rng.choice(["-1", "99999999999999999999", "2147483648", "1e9", "0.5", "9223372036854775807"]) + s[m.end():]
                b = bytearray(s.encode("latin1"))
            g = ctypes.c_void_p()
            rc = L.pccl_graph_load_json(bytes(b), len(b), ctypes.byref(g))
            if rc != 0:
                failed += 1
                assert rc < 0 and L.pccl_hip_last_error()
                continue
            loaded += 1
            arr = (ctypes.c_void_p * 2)(g, g)
            p = ctypes.c_void_p()
            if L.pccl_program_link(arr, 2, ctypes.byref(p)) == 0:
                L.pccl_program_free(p)
            L.pccl_graph_free(g)
    assert failed > 50 and loaded > 10


def test_bench_finds_the_committed_counter_figures():
    """bench.py copies the counter-measured HBM bytes per launch of its kernel from the committed
    rocprofv3 summary of the same workload and names that file (`roofline.traffic_source`): the files
    it looks for exist, hold a positive byte count, sit beside a summary that names their kernel and
    quotes that count, and record the hash of the kernel source they were taken on - a figure from another version of the
    kernels is not handed on."""
    import hashlib
    import importlib.util
    import json
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    spec = importlib.util.spec_from_file_location("bench_under_test", os.path.join(root, "bench.py"))
    bench = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(bench)
    current = hashlib.sha256(open(os.path.join(root, "pccl_amd", "csrc", "kernels.hip"), "rb").read()).hexdigest()
    assert bench.kernel_source_sha256() == current
    allreduces = ["ring_allreduce_R8_bf16_512MiB", "rhd_allreduce_R16_f32_64MiB", "tree_allreduce_R32_int32_sum_96MiB", "tree_allreduce_R32_f32_max_96MiB"]
    wanted = [(k, stem) for k in ("phased_kernel", "column_slot_kernel") for stem in allreduces]
    wanted += [("level_kernel", "ring_allreduce_R8_bf16_512MiB"), ("persistent_kernel", "ring_allreduce_R8_bf16_512MiB"),
               ("phased_kernel", "ring_reduce_scatter_R8_f16_512MB_staged"), ("phased_kernel", "ring_allgather_R8_f16_512MB_staged")]
    for kernel, stem in wanted:
        path = os.path.join(root, "profiles", f"{kernel}_{stem}.traffic.json")
        rec = json.load(open(path))
        assert rec["hbm_bytes_per_launch"] > 0 and len(rec["kernels_hip_sha256"]) == 64, (kernel, stem)
        nbytes, rel = bench.committed_traffic(kernel, stem)
        if rec["kernels_hip_sha256"] == current:
            assert rel == f"profiles/{kernel}_{stem}.traffic.json" and nbytes == rec["hbm_bytes_per_launch"], (kernel, stem)
        else:
            assert nbytes is None and rel.startswith(f"profiles/{kernel}_{stem}.traffic.json") and "not used" in rel
        summary = os.path.join(root, "profiles", f"{kernel}_{stem}.md")
        assert os.path.exists(summary) and kernel in open(summary).read()
        # the summary quotes the byte count that the file holds (they are written together)
        assert f"{rec['hbm_bytes_per_launch']:,}" in open(summary).read(), (kernel, stem)
    assert bench.committed_traffic("column_slot_kernel", None) == (None, None)
    assert bench.committed_traffic("column_slot_kernel", "no_such_workload") == (None, None)
