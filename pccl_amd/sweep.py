"""Timing sweep over the benchmark configurations other than the headline one.

    python -m pccl_amd.sweep [--config c3|c4|c5|all] [--mode auto|column|stepwise] [--reps N]
                             [--option KEY=VALUE ...] [--prepared]

Prints one JSON line per measurement: kernel time by HIP events on the launch stream, algorithmic
bytes (reduce 3*n*esize, copy 2*n*esize summed over the linked program) and GB/s.  Inputs are drawn
on the GPU; results are not checked here (tests/test_gpu_configs.py does that on the same graphs).

c3  recursive halving-doubling allreduce, 16 ranks, 64 MiB f32 per rank, 2 channels (in place)
c4  ring reduce_scatter and allgather, 8 ranks, fp16, 4 KB .. 256 MB (x4) and 512 MB per rank
    (staged calls, the reference's call shape: the staging copies are part of the time)
c5  binary-tree allreduce, 32 ranks, 96 MiB per rank, int32 SUM and f32 MAX, every op cut into 8
    ragged pieces whose boundaries are off 16-byte alignment (in place)
"""
from __future__ import annotations

import argparse
import json
import sys

import torch

from .dsl import ALGORITHMS, compile_to_json_string, ragged_cuts
from .engine import Engine

TD = {"float32": torch.float32, "float16": torch.float16, "bfloat16": torch.bfloat16, "int32": torch.int32}


def graphs(alg, method, world, n, dtype, channels, **ext):
    a = ALGORITHMS[alg]()
    return [compile_to_json_string(getattr(a, method)(r, world, n, dtype=dtype, executor="sm",
                                                      num_channels=channels, **ext)) for r in range(world)]


def timed(fn, reps):
    fn()
    torch.cuda.synchronize()
    ev = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(reps)]
    for a, b in ev:
        a.record()
        fn()
        b.record()
    torch.cuda.synchronize()
    ms = sorted(a.elapsed_time(b) for a, b in ev)
    return ms[len(ms) // 2], ms[0]


OPTIONS: list = []   # (key, value) engine options applied to every case
PREPARED = False     # staged cases through Engine.prepare (argument arrays built once)


def run_case(label, world, jsons, make_in, out_elems, mode, reps, inplace):
    eng = Engine(world, 0)
    try:
        for r, j in enumerate(jsons):
            eng.register_operation_json("op", j, r)
        eng.set_option("mode", mode)
        for key, val in OPTIONS:
            eng.set_option(key, val)
        info = eng.op_info("op")
        x = make_in()
        if inplace:
            med, best = timed(lambda: eng.execute_inplace("op", x), reps)
        else:
            outs = [torch.empty(out_elems, dtype=x[0].dtype, device="cuda") for _ in range(world)]
            call = eng.prepare("op", x, outs) if PREPARED else (lambda: eng.execute_operation_async("op", x, outs))
            med, best = timed(call, reps)
        b = info["algorithmic_bytes"]
        print(json.dumps({"case": label, "mode": mode, "in_place": inplace, "levels": info["num_levels"],
                          "data_ops": info["num_data_ops"], "algorithmic_bytes": b,
                          "ms_median": round(med, 4), "ms_min": round(best, 4),
                          "GB/s": round(b / (med * 1e-3) / 1e9, 1),
                          "planned_traffic_bytes": (info["column_load_bytes"] + info["column_store_bytes"]) if inplace
                          else (info["staged_load_bytes"] + info["staged_store_bytes"])}),
              flush=True)
    finally:
        eng.close()


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--config", default="all")
    ap.add_argument("--mode", default="auto")
    ap.add_argument("--reps", type=int, default=20)
    ap.add_argument("--option", action="append", default=[], metavar="KEY=VALUE",
                    help="engine option for every case (e.g. lds_slots=0); repeatable")
    ap.add_argument("--prepared", action="store_true",
                    help="issue the staged calls (c4) through Engine.prepare: only the C call per invocation")
    args = ap.parse_args()
    global PREPARED
    PREPARED = args.prepared
    for kv in args.option:
        key, _, val = kv.partition("=")
        OPTIONS.append((key, val))
    g = torch.Generator(device="cuda").manual_seed(0)
    want = args.config

    if want in ("c3", "all"):
        world, n = 16, 16_777_216
        run_case("c3 rhd allreduce R16 f32 64MiB 2ch", world, graphs("rhd", "build_allreduce", world, n, "float32", 2),
                 lambda: [torch.rand(n, generator=g, device="cuda") * 2 - 1 for _ in range(world)], n,
                 args.mode, args.reps, True)
    if want in ("c4", "all"):
        world = 8
        sizes = [4096 * 4 ** k for k in range(9)] + [512 << 20]
        for nbytes in sizes:
            n = nbytes // 2
            chunk = n // world
            for method, in_elems, out_elems in (("build_reduce_scatter", n, chunk), ("build_allgather", chunk, n)):
                run_case(f"c4 ring {method[6:]} R8 f16 {nbytes} B/rank", world,
                         graphs("ring", method, world, n, "float16", 1),
                         lambda: [(torch.randn(in_elems, generator=g, device="cuda") * 0.1).half() for _ in range(world)],
                         out_elems, args.mode, args.reps, False)
    if want in ("c5", "all"):
        world, n = 32, 25_165_824
        cuts = ragged_cuts(n, 8, seed=0)
        run_case("c5 tree allreduce R32 int32 sum 96MiB ragged", world,
                 graphs("tree", "build_allreduce", world, n, "int32", 1, reduce_op="sum", cuts=cuts),
                 lambda: [torch.randint(-1000, 1000, (n,), generator=g, device="cuda", dtype=torch.int32) for _ in range(world)],
                 n, args.mode, args.reps, True)
        run_case("c5 tree allreduce R32 f32 max 96MiB ragged", world,
                 graphs("tree", "build_allreduce", world, n, "float32", 1, reduce_op="max", cuts=cuts),
                 lambda: [torch.randn(n, generator=g, device="cuda") for _ in range(world)],
                 n, args.mode, args.reps, True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
