"""Counting semaphores across executions and operations.  The reference keeps one signal region per
engine, shared by every registered operation and cleared only by Engine::resetSignals
(csrc/engine_c.cc:131-146, 576-593); a wait passes on a count above zero and takes one
(csrc/plugins/cuda/cuda_executor.cu:425-445).  So a notify that no wait consumed is found by the next
execution that waits on that semaphore.  The engine tracks those counts on the host and links each
operation for the counts it finds; checked here against the CPU oracle run with the same state."""
import json

import numpy as np
import pytest
import torch

from helpers import bits_equal, carry_expected, carry_ops, mismatch_report, oracle
from pccl_amd._lib import ERR_INVALID, ERR_LINK, PcclError

pytestmark = pytest.mark.gpu


def _engine(engine_factory, n, mode):
    eng = engine_factory(2)
    eng.set_option("mode", mode)
    jsons = carry_ops(n)
    for name, js in jsons.items():
        for r, j in enumerate(js):
            eng.register_operation_json(name, j, r)
    return eng, {k: [oracle.Graph(json.loads(j)) for j in v] for k, v in jsons.items()}


def _state(sig):
    return {(int(r), int(i)): int(sig[r, i]) for r, i in zip(*np.nonzero(sig))}


@pytest.mark.parametrize("mode", ["auto", "stepwise", "persistent"])
@pytest.mark.parametrize("n", [64, 300000])
def test_counts_left_by_one_execution_are_found_by_the_next(engine_factory, mode, n):
    eng, og = _engine(engine_factory, n, mode)
    try:
        rng = np.random.default_rng(n)
        host = [rng.standard_normal(n).astype(np.float32) for _ in range(2)]
        bufs = [torch.from_numpy(h.copy()).cuda() for h in host]
        sig = oracle.new_signals(2)

        def step(name, staged=False):
            nonlocal bufs
            print(f"{mode} n={n}: {name} staged={staged} on {eng.signals()}", flush=True)
            closed = carry_expected(name, host)
            oracle.run(og[name], host, signals=sig)
            for h, c in zip(host, closed):        # the oracle against the operation's description
                assert np.array_equal(h.view(np.int32), c.view(np.int32))
            if staged:
                bufs = eng.execute_operation(name, bufs)
            else:
                eng.execute_inplace(name, bufs, sync=True)
            for r in range(2):
                want = torch.from_numpy(host[r])
                assert bits_equal(bufs[r], want), f"{name}, rank {r}: {mismatch_report(bufs[r], want)}"
            assert eng.signals() == _state(sig), name

        def deadlocks(name):
            before = [b.clone() for b in bufs]
            with pytest.raises(PcclError) as e:
                eng.execute_inplace(name, bufs, sync=True)
            assert e.value.code == ERR_LINK and "deadlock" in str(e.value) and "signal 5" in str(e.value)
            assert all(bits_equal(a, b) for a, b in zip(before, bufs))      # nothing ran
            assert eng.signals() == _state(sig)                             # and nothing was counted

        assert eng.signals() == {}
        deadlocks("take")                          # from zero nobody lets rank 1's wait through
        step("give")
        assert eng.signals() == {(1, 5): 1}
        step("take", staged=True)                  # runs on the count that `give` left
        assert eng.signals() == {}
        deadlocks("take")
        for k in range(1, 4):
            step("give", staged=(k == 2))
            assert eng.signals() == {(1, 5): k}
        assert eng.op_info("give")["residual_signals"] == 1 and eng.op_info("take")["residual_signals"] == 1
        # `pair` is race-free from zero; on a carried count its wait passes before its notify
        with pytest.raises(PcclError) as e:
            eng.execute_inplace("pair", bufs, sync=True)
        assert e.value.code == ERR_LINK and "data race" in str(e.value)
        assert eng.signals() == {(1, 5): 3}
        for k in (2, 1, 0):
            step("take")
        assert eng.signals() == {}
        assert eng.op_info("pair")["residual_signals"] == 0
        step("pair")                               # linked again for the counts it finds now: none
        step("pair", staged=True)
        # reset_signals clears the whole region, whichever operation is named
        step("give"); step("give")
        eng.reset_signals("pair")
        sig[:] = 0
        assert eng.signals() == {}
        deadlocks("take")
        step("pair")
    finally:
        eng.reset_signals("give")
        eng.set_option("mode", "auto")


def test_operations_that_move_counts_are_not_recorded_into_graphs(engine_factory):
    """A recorded launch is replayed without the host, which could not follow the counts: refused with
    a message that says so.  A balanced operation on untouched semaphores records as before."""
    n = 4096
    eng, _ = _engine(engine_factory, n, "auto")
    try:
        bufs = [torch.randn(n, device="cuda") for _ in range(2)]
        eng.execute_inplace("pair", bufs, sync=True)          # linked and uploaded outside the capture
        eng.execute_inplace("give", bufs, sync=True)
        eng.reset_signals("give")
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        graph = torch.cuda.CUDAGraph()
        seen = []
        with torch.cuda.stream(side):
            with torch.cuda.graph(graph, stream=side):
                eng.execute_inplace("pair", bufs)
                try:
                    eng.execute_inplace("give", bufs)
                except PcclError as e:
                    seen.append(e)
        torch.cuda.current_stream().wait_stream(side)
        assert len(seen) == 1 and seen[0].code == ERR_INVALID and "carry counts" in str(seen[0])
        assert eng.signals() == {}
        start = [b.clone() for b in bufs]
        graph.replay()
        torch.cuda.synchronize()
        want = carry_expected("pair", [s.cpu().numpy() for s in start])
        for r in range(2):
            assert bits_equal(bufs[r], torch.from_numpy(want[r]))
    finally:
        eng.reset_signals("give")


def test_counts_through_the_entry_point_that_allocates_nothing(engine_factory):
    n = 4096
    eng, og = _engine(engine_factory, n, "auto")
    try:
        rng = np.random.default_rng(3)
        host = [rng.standard_normal(n).astype(np.float32) for _ in range(2)]
        bufs = [torch.from_numpy(h.copy()).cuda() for h in host]
        sig = oracle.new_signals(2)
        for name in ("give", "give", "take", "pair", "take"):
            if name == "pair":                     # a data race while a count is there
                with pytest.raises(PcclError) as e:
                    eng.execute_inplace_static(name, bufs, sync=True)
                assert e.value.code == ERR_LINK and "data race" in str(e.value)
                continue
            oracle.run(og[name], host, signals=sig)
            eng.execute_inplace_static(name, bufs, sync=True)
            for r in range(2):
                assert bits_equal(bufs[r], torch.from_numpy(host[r])), name
            assert eng.signals() == _state(sig)
        assert eng.signals() == {}
        # an operation whose tables are on the device and whose counts have changed would have to be
        # linked again, which frees device memory: this entry point says so instead
        eng.execute_inplace("pair", bufs, sync=True)
        eng.execute_inplace("give", bufs, sync=True)
        with pytest.raises(PcclError) as e:
            eng.execute_inplace_static("pair", bufs, sync=True)
        assert e.value.code == ERR_INVALID and "frees nothing" in str(e.value)
    finally:
        eng.reset_signals("give")
