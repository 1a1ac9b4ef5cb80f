#!/usr/bin/env python3
"""Headline benchmark: the 8-virtual-rank, 512 MB-per-rank bf16 ring-allreduce graph on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--mode auto|column|stepwise]

A step is one execution of the compiled graph (448 data ops over 8 rank buffers resident in HBM),
in place on the rank buffers, one launch of the column runner.  Prints ONE JSON line.

* value     algorithmic schedule bytes (reduce 3*n*esize, copy 2*n*esize, summed over the linked
            program = 5*(R-1)*S) times K, divided by the wall time of the K timed steps
* roofline  the same bytes divided by the average kernel duration measured with HIP events on the
            launch stream (torch's current stream, which is the stream the C ABI launches on),
            against the 8 TB/s HBM peak; `traffic` is the measured HBM bytes per launch from the
            committed rocprofv3 counter summary when present
* cpu_baseline  the CPU oracle (oracle/, OpenMP) executing the same graph shape on a bounded sample
            on this box's host cores; a reported baseline, not the target

Inputs: one CPU generator seeded 0; for rank r = 0..7, for slice s = 0..7, draw
torch.randn(N/8) and cast to bf16 (rank-major, slice-major) — N(0,1) values as the configuration
prescribes, generated in slices to bound host memory.  The first execution is verified at full size
before anything is timed: all ranks must hold bit-identical results and those must equal the
ring's per-element reduction order evaluated with plain torch bf16 adds.
"""
from __future__ import annotations

import argparse
import hashlib
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

R = 8
N = 268_435_456          # bf16 elements per rank = 512 MiB
CHANNELS = 4
DTYPE = "bfloat16"
PEAK_GBPS = 8000.0
WORKLOAD = "ring_allreduce_sum_R8_bf16_512MiB_per_rank_4ch"


def log(msg: str) -> None:
    print(f"[bench] {msg}", file=sys.stderr, flush=True)


def build_graphs(n: int, channels: int):
    from pccl_amd.dsl import RingAllreduce, compile_to_json_string
    return [compile_to_json_string(RingAllreduce().build_allreduce(r, R, n, dtype=DTYPE, executor="sm",
                                                                   num_channels=channels))
            for r in range(R)]


def make_inputs(n: int, device):
    import torch
    g = torch.Generator().manual_seed(0)
    slices = 8
    per = n // slices
    bufs = []
    for r in range(R):
        buf = torch.empty(n, dtype=torch.bfloat16, device=device)
        for s in range(slices):
            buf[s * per:(s + 1) * per] = torch.randn(per, generator=g).to(torch.bfloat16).to(device)
        bufs.append(buf)
    return bufs


def ring_expected(inputs, n: int, channels: int):
    """Ring order (chunk c of channel ch: acc = x_c; acc = x_(c+k) + acc, k = 1..R-1), each add
    rounded to bf16, evaluated with torch's own bf16 add on the GPU."""
    import torch
    per_ch = n // channels
    per_rank = per_ch // R
    out = torch.empty_like(inputs[0])
    for ch in range(channels):
        for c in range(R):
            lo = ch * per_ch + c * per_rank
            acc = inputs[c][lo:lo + per_rank].clone()
            for k in range(1, R):
                acc = inputs[(c + k) % R][lo:lo + per_rank] + acc
            out[lo:lo + per_rank] = acc
    return out


def sha256_of(t) -> str:
    import torch
    h = hashlib.sha256()
    flat = t.view(torch.int16)
    step = 1 << 26
    for i in range(0, flat.numel(), step):
        h.update(flat[i:i + step].cpu().numpy().tobytes())
    return h.hexdigest()


def device_info(dev) -> dict:
    """Name, CU count and - best effort, from the driver's sysfs files - the current clocks and the
    power cap of the GPU (no helper program is started: a process that holds the GPU must not)."""
    import glob
    import re
    import torch
    props = torch.cuda.get_device_properties(dev)
    info = {"name": props.name, "compute_units": props.multi_processor_count,
            "hbm_gib": round(props.total_memory / 2**30, 1), "sclk_mhz": None, "mclk_mhz": None, "power_cap_w": None}

    def current_level(pattern):
        for path in sorted(glob.glob(pattern)):
            try:
                with open(path) as f:
                    for line in f:
                        m = re.match(r"\s*\d+:\s*(\d+)Mhz\s*\*", line)
                        if m:
                            return float(m.group(1))
            except OSError:
                pass
        return None

    info["sclk_mhz"] = current_level("/sys/class/drm/card*/device/pp_dpm_sclk")
    info["mclk_mhz"] = current_level("/sys/class/drm/card*/device/pp_dpm_mclk")
    for path in sorted(glob.glob("/sys/class/drm/card*/device/hwmon/hwmon*/power1_cap")):
        try:
            with open(path) as f:
                info["power_cap_w"] = int(f.read().strip()) / 1e6
            break
        except (OSError, ValueError):
            pass
    return info


def cpu_baseline(sample_elems: int, channels: int, reps: int = 3):
    """Time the CPU oracle on the same graph shape at `sample_elems` elements per rank."""
    import numpy as np
    from oracle import oracle
    graphs = [oracle.Graph(json.loads(j)) for j in build_graphs(sample_elems, channels)]
    rng = np.random.default_rng(0)
    threads = os.cpu_count() or 1
    env = os.environ.get("OMP_NUM_THREADS")
    if env and env.isdigit():
        threads = int(env)
    # first touch by filling; bf16 bit patterns of N(0,1)-like magnitudes
    bufs = [(rng.integers(0x3C00, 0x4000, sample_elems, dtype=np.uint16)) for _ in range(R)]
    stats = oracle.run(graphs, bufs, threads=threads)      # warm-up
    times = []
    for _ in range(reps):
        t0 = time.perf_counter()
        stats = oracle.run(graphs, bufs, threads=threads)
        times.append(time.perf_counter() - t0)
    times.sort()
    med = times[len(times) // 2]
    model = ""
    try:
        with open("/proc/cpuinfo") as f:
            model = next((line.split(":", 1)[1].strip() for line in f if line.startswith("model name")), "")
    except OSError:
        pass
    return {"value": round(stats.bytes / med / 1e9, 2), "unit": "GB/s", "cores": threads, "kind": "port",
            "cpu_model": model, "host_cpus_visible": os.cpu_count(),
            "sample": f"same ring graph (R={R}, {channels} channels, bf16) at {sample_elems} elements "
                      f"per rank ({sample_elems * 2 >> 20} MiB), {stats.bytes} algorithmic bytes, median of "
                      f"{reps} runs after 1 warm-up, {med * 1e3:.1f} ms"}


def measured_traffic(mode: str, levels: int):
    """HBM bytes per execution of the headline graph from the committed rocprofv3 counter summaries
    (FETCH_SIZE + WRITE_SIZE scaled by a 1 GiB copy): one launch of the column kernel, or one launch
    per dependency level of the level kernel."""
    if mode == "persistent":
        return None
    kernel = "level_kernel" if mode == "stepwise" else "column_slot_kernel"
    path = os.path.join(ROOT, "profiles", f"{kernel}_ring_allreduce_R8_bf16_512MiB.traffic.json")
    try:
        with open(path) as f:
            per_launch = json.load(f).get("hbm_bytes_per_launch")
    except (OSError, ValueError):
        return None
    if per_launch is None:
        return None
    return per_launch * levels if mode == "stepwise" else per_launch


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--mode", default="auto")
    ap.add_argument("--elems", type=int, default=N, help="elements per rank (default: the headline size)")
    ap.add_argument("--channels", type=int, default=CHANNELS)
    ap.add_argument("--vecs-per-thread", type=int, default=0)
    ap.add_argument("--num-blocks", type=int, default=-1)
    ap.add_argument("--option", action="append", default=[], metavar="KEY=VALUE",
                    help="engine option to set before the run (e.g. lds_slots=0, slot_threads=128); repeatable")
    ap.add_argument("--rank-skew-bytes", type=int, default=0,
                    help="carve the rank buffers out of one allocation, each this many bytes further in than its size")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-verify", action="store_true")
    ap.add_argument("--gpu-inputs", action="store_true",
                    help="draw the inputs with the GPU generator (tuning sweeps only; not the prescribed inputs)")
    ap.add_argument("--cpu-sample-elems", type=int, default=N)
    ap.add_argument("--cpu-reps", type=int, default=60)
    ap.add_argument("--calibrate-copy-bytes", type=int, default=0,
                    help="also launch the library's plain copy kernel on this many bytes (3 times): a "
                         "known-traffic reference for scaling rocprofv3 FETCH_SIZE / WRITE_SIZE")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on one GPU: the R ranks are virtual ranks resident in one "
              "MI355X's HBM and no multi-GPU path exists; run with --gpus 1", file=sys.stderr)
        return 2

    import torch
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible; the executor has no CPU fallback", file=sys.stderr)
        return 1
    from pccl_amd.engine import Engine

    n, channels = args.elems, args.channels
    dev = torch.device("cuda", 0)
    eng = Engine(R, 0)
    for r, text in enumerate(build_graphs(n, channels)):
        eng.register_operation_json("bench", text, r)
    eng.set_option("mode", args.mode)
    if args.vecs_per_thread:
        eng.set_option("vecs_per_thread", args.vecs_per_thread)
    if args.num_blocks >= 0:
        eng.set_option("num_blocks", args.num_blocks)
    for kv in args.option:
        key, _, val = kv.partition("=")
        eng.set_option(key, val)
    info = eng.op_info("bench")
    alg_bytes = info["algorithmic_bytes"]
    log(f"program: {info}")

    t0 = time.perf_counter()
    if args.gpu_inputs:
        torch.manual_seed(0)
        pristine = [torch.randn(n, device=dev, dtype=torch.float32).to(torch.bfloat16) for _ in range(R)]
    else:
        pristine = make_inputs(n, dev)
    log(f"inputs generated in {time.perf_counter() - t0:.1f} s")
    if args.rank_skew_bytes:
        # rank buffers carved out of one allocation, rank r starting r * (size + skew) bytes in: the
        # same position of different ranks then falls on different memory channels
        stride = n + args.rank_skew_bytes // 2
        arena = torch.empty(R * stride, dtype=torch.bfloat16, device=dev)
        bufs = [arena[r * stride:r * stride + n] for r in range(R)]
        for b, p in zip(bufs, pristine):
            b.copy_(p)
        log("rank buffer addresses: " + " ".join(hex(b.data_ptr()) for b in bufs))
    else:
        bufs = [p.clone() for p in pristine]
        log("rank buffer addresses: " + " ".join(hex(b.data_ptr()) for b in bufs))

    # the first execution in the process (tables just uploaded, nothing of the buffers in any cache)
    c0, c1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    c0.record()
    eng.execute_inplace("bench", bufs)
    c1.record()
    torch.cuda.synchronize()
    cold_ms = c0.elapsed_time(c1)

    verify = {}
    if not args.no_verify:
        same = all(torch.equal(bufs[0].view(torch.int16), b.view(torch.int16)) for b in bufs[1:])
        want = ring_expected(pristine, n, channels)
        exact = torch.equal(want.view(torch.int16), bufs[0].view(torch.int16))
        ref32 = sum(p[:1 << 20].float() for p in pristine)
        rel = ((bufs[0][:1 << 20].float() - ref32).abs() / ref32.abs().clamp_min(1.0)).max().item()
        verify = {"ranks_identical": bool(same), "matches_ring_order_bf16": bool(exact),
                  "max_rel_err_vs_fp32_sum_first_1Mi": round(rel, 5), "output_sha256": sha256_of(bufs[0])}
        # at the headline size with the prescribed inputs: the hashes committed with the tests (the
        # output hash is what the CPU oracle computes at full size, tests/golden/make_headline_sha256.py)
        golden_path = os.path.join(ROOT, "tests", "golden", "headline_sha256.json")
        if n == N and channels == CHANNELS and not args.gpu_inputs and os.path.exists(golden_path):
            golden = json.load(open(golden_path))
            verify["input_rank0_matches_committed_sha256"] = sha256_of(pristine[0]) == golden["input_sha256_per_rank"][0]
            verify["output_matches_committed_oracle_sha256"] = verify["output_sha256"] == golden["output_sha256"]
            exact = exact and verify["input_rank0_matches_committed_sha256"] and verify["output_matches_committed_oracle_sha256"]
        log(f"verify: {verify}")
        del want
        if not (same and exact):
            print(json.dumps({"error": "verification failed", **verify}))
            return 1
        for b, p in zip(bufs, pristine):
            b.copy_(p)

    if args.calibrate_copy_bytes:
        from pccl_amd import _lib
        src = torch.empty(args.calibrate_copy_bytes, dtype=torch.uint8, device=dev).random_(0, 256)
        dst = torch.empty_like(src)
        for _ in range(3):
            _lib.check(_lib.lib().pccl_hip_copy(3, src.data_ptr(), dst.data_ptr(), src.numel(), None))
        torch.cuda.synchronize()
        del src, dst

    for _ in range(args.warmup):
        eng.execute_inplace("bench", bufs)
    torch.cuda.synchronize()
    ev0 = [torch.cuda.Event(enable_timing=True) for _ in range(args.steps)]
    ev1 = [torch.cuda.Event(enable_timing=True) for _ in range(args.steps)]
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(args.steps):
        ev0[i].record()
        eng.execute_inplace("bench", bufs)
        ev1[i].record()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    kern_ms = [a.elapsed_time(b) for a, b in zip(ev0, ev1)]
    avg_ms = sum(kern_ms) / len(kern_ms)
    ms_per_step = wall * 1e3 / args.steps
    value = alg_bytes / (ms_per_step * 1e-3) / 1e9
    achieved = alg_bytes / (avg_ms * 1e-3) / 1e9

    # end to end the reference's way: input and output staging copies included
    outs = [torch.empty_like(p) for p in pristine]
    eng.execute_operation("bench", pristine, outs)
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    reps = max(3, args.steps // 4)
    for _ in range(reps):
        eng.execute_operation_async("bench", pristine, outs)
    e1.record()
    torch.cuda.synchronize()
    staged_ms = e0.elapsed_time(e1) / reps
    del outs

    # the same graph op by op (one launch per dependency level, every op moving its full bytes)
    op_by_op = None
    if args.mode == "auto":
        eng.set_option("mode", "stepwise")
        for _ in range(2):
            eng.execute_inplace("bench", bufs)
        torch.cuda.synchronize()
        e0.record()
        for _ in range(reps):
            eng.execute_inplace("bench", bufs)
        e1.record()
        torch.cuda.synchronize()
        sw_ms = e0.elapsed_time(e1) / reps
        eng.set_option("mode", "auto")
        op_by_op = {"mode": "stepwise", "ms_per_step": round(sw_ms, 4), "GB/s": round(alg_bytes / (sw_ms * 1e-3) / 1e9, 1),
                    "frac_of_hbm_peak": round(alg_bytes / (sw_ms * 1e-3) / 1e9 / PEAK_GBPS, 4),
                    "note": "HBM traffic equals the algorithmic bytes in this mode (profiles/level_kernel_*.md)"}

    # and as one persistent launch whose workgroups order themselves through device-side flags
    persistent = None
    if args.mode == "auto":
        eng.set_option("mode", "persistent")
        for _ in range(2):
            eng.execute_inplace("bench", bufs)
        torch.cuda.synchronize()
        e0.record()
        for _ in range(reps):
            eng.execute_inplace("bench", bufs)
        e1.record()
        torch.cuda.synchronize()
        pm_ms = e0.elapsed_time(e1) / reps
        eng.sync_operation("bench")      # would raise if a bounded wait had expired
        eng.set_option("mode", "auto")
        persistent = {"mode": "persistent", "ms_per_step": round(pm_ms, 4), "GB/s": round(alg_bytes / (pm_ms * 1e-3) / 1e9, 1),
                      "frac_of_hbm_peak": round(alg_bytes / (pm_ms * 1e-3) / 1e9 / PEAK_GBPS, 4),
                      "note": "one launch for the whole graph, every op moving its full bytes, ordering by device-side flags (one per work item, one ready word per op)"}

    default_runner = not any(kv.split("=")[0] in ("lds_slots", "slot_threads", "slot_direct") for kv in args.option)
    traffic = measured_traffic(args.mode, info["num_levels"]) if (n == N and channels == CHANNELS and default_runner) else None
    result = {
        "metric": "HBM GB/s (algorithmic schedule bytes read+written per second), 8-vrank 512MB bf16 ring allreduce graph",
        "value": round(value, 1), "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"workload": WORKLOAD if (n == N and channels == CHANNELS) else
                   f"ring_allreduce_sum_R8_bf16_{n}elems_per_rank_{channels}ch",
                   "virtual_ranks": R, "bytes_per_rank": n * 2, "channels": channels, "data_ops": info["num_data_ops"],
                   "algorithmic_bytes_per_step": alg_bytes, "mode": args.mode, "in_place": True},
        "pct_of_hbm_peak": round(100 * value / PEAK_GBPS, 1),
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": PEAK_GBPS, "unit": "GB/s",
                     "frac": round(achieved / PEAK_GBPS, 4), "traffic": traffic,
                     "kernel_ms_avg": round(avg_ms, 4), "kernel_ms_min": round(min(kern_ms), 4),
                     "kernel_ms_median": round(sorted(kern_ms)[len(kern_ms) // 2], 4),
                     "kernel_ms_first_execution": round(cold_ms, 4),
                     "planned_load_bytes": info["column_load_bytes"], "planned_store_bytes": info["column_store_bytes"]},
        "end_to_end_staged": {"ms_per_call": round(staged_ms, 4), "GB/s": round(alg_bytes / (staged_ms * 1e-3) / 1e9, 1),
                              "note": "the reference's call shape (separate input and output tensors per rank, execute_operation_async); "
                                      "the staging copies are fused into the program, so this is again one launch"},
        "op_by_op": op_by_op,
        "single_launch_flag_ordered": persistent,
        "device": device_info(dev),
        "verify": verify,
    }
    if result["roofline"]["frac"] > 1:
        result["roofline"]["note"] = ("achieved counts the schedule's algorithmic bytes (35 S); the column runner executes "
                                      "the same ops with 16 S of HBM traffic (forwarded values and re-read partial results "
                                      "stay in registers and LDS), so hbm_frac, not frac, is the memory system's utilisation")
    if args.gpu_inputs:
        result["data"] = "synthetic (GPU generator: tuning run)"
    if traffic:
        result["roofline"]["hbm_frac"] = round(traffic / (avg_ms * 1e-3) / 1e9 / PEAK_GBPS, 4)
    if not args.no_cpu_baseline:
        del bufs, pristine
        torch.cuda.empty_cache()
        result["cpu_baseline"] = cpu_baseline(min(args.cpu_sample_elems, n), channels, args.cpu_reps)
    print(json.dumps(result))
    eng.close()
    return 0


if __name__ == "__main__":
    sys.exit(main())
