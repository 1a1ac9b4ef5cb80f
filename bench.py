#!/usr/bin/env python3
"""Benchmark of the executor on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--config c2|c3|c4|c5] [--mode auto|column|stepwise|persistent]

The default (``--config c2``) is the headline: the 8-virtual-rank, 512 MiB-per-rank bf16 ring-allreduce
graph (4 channels, 448 data ops), in place on 8 rank buffers resident in HBM.  A step is one
execution of the compiled graph.  Prints ONE JSON line (``c4`` prints one per message size and
collective).

* value      HBM bytes the step actually moves, divided by the wall time per step.  For the column
             runner these are the bytes its plan loads and stores (every rank buffer read once and
             written once: 16 S for the headline), which the committed rocprofv3 FETCH_SIZE /
             WRITE_SIZE figures confirm; for the level and persistent runners every op moves its
             full bytes, so the figure is the algorithmic byte count (5 (R-1) S).
* roofline   the same bytes divided by the average kernel duration measured with HIP events on the
             launch stream (torch's current stream, which is the stream the C ABI launches on),
             against the 8 TB/s HBM peak.  ``traffic`` is the counter-measured figure of the
             profile named in ``traffic_source`` (null where no profile covers the run).
* algorithmic_equiv_GBps   the schedule's algorithmic bytes (reduce 3 n esize, copy 2 n esize over the
             linked program) per second: what a runner that executes op by op would have to
             sustain to be as fast.  Not an HBM rate.
* cpu_baseline   the CPU oracle (oracle/, OpenMP) executing the same graph on this box's host
             cores; a reported baseline, not the target
* other_configs  (plain default run only, after the headline has been measured) configurations 3, 5
             with both element types and the 512 MB pair of 4, each verified at full size and timed
             the same way: ms per step, HBM bytes and rate, fraction of peak, and the per-rank
             alg_bw / bus_bw of the reference's own bandwidth script

Other configurations: c3 = recursive halving-doubling allreduce, 16 ranks, 64 MiB f32, 2 channels;
c4 = ring reduce_scatter and allgather, 8 ranks, fp16, 4 KB to 512 MB per rank as staged calls;
c5 = binary-tree allreduce, 32 ranks, 96 MiB per rank, int32 SUM and f32 MAX (``--c5-dtype``), every
op cut into 8 ragged pieces off 16-byte alignment.

Headline inputs: one CPU generator seeded 0; for rank r = 0..7, for slice s = 0..7, draw
torch.randn(N/8) and cast to bf16 (rank-major, slice-major) - N(0,1) values as the configuration
prescribes, generated in slices to bound host memory.  The first execution is verified at full size
before anything is timed: all ranks must hold bit-identical results, those must equal the ring's
per-element reduction order evaluated with plain torch bf16 adds, and their sha256 must be the
one the CPU oracle produced (tests/golden/headline_sha256.json).
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

PEAK_GBPS = 8000.0
METRIC = "HBM GB/s & % of 8 TB/s peak (bytes read+written per second)"


def log(msg: str) -> None:
    print(f"[bench] {msg}", file=sys.stderr, flush=True)


# ----------------------------------------------------------------------------------------- workloads

def graphs(alg: str, method: str, world: int, n: int, dtype: str, channels: int, **ext):
    from pccl_amd.dsl import ALGORITHMS, compile_to_json_string
    a = ALGORITHMS[alg]()
    return [compile_to_json_string(getattr(a, method)(r, world, n, dtype=dtype, executor="sm",
                                                      num_channels=channels, **ext)) for r in range(world)]


def headline_inputs(n: int, world: int, device):
    import torch
    g = torch.Generator().manual_seed(0)
    slices = 8
    per = n // slices
    bufs = []
    for _ in range(world):
        buf = torch.empty(n, dtype=torch.bfloat16, device=device)
        for s in range(slices):
            buf[s * per:(s + 1) * per] = torch.randn(per, generator=g).to(torch.bfloat16).to(device)
        bufs.append(buf)
    return bufs


def ring_expected(inputs, n: int, channels: int):
    """Ring order (chunk c of channel ch: acc = x_c; acc = x_(c+k) + acc, k = 1..R-1), each add
    rounded to the storage type, evaluated with torch's own adds on the GPU."""
    import torch
    world = len(inputs)
    per_ch = n // channels
    per_rank = per_ch // world
    out = torch.empty_like(inputs[0])
    for ch in range(channels):
        for c in range(world):
            lo = ch * per_ch + c * per_rank
            acc = inputs[c][lo:lo + per_rank].clone()
            for k in range(1, world):
                acc = inputs[(c + k) % world][lo:lo + per_rank] + acc
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


class Workload:
    """One configuration: graphs, inputs, how to check a result, which profile measured its traffic."""

    def __init__(self, key, name, world, n, dtype, jsons, make_inputs, check, traffic_stem=None, channels=1):
        self.key, self.name, self.world, self.n, self.dtype = key, name, world, n, dtype
        self.jsons, self.make_inputs, self.check, self.traffic_stem, self.channels = jsons, make_inputs, check, traffic_stem, channels


def workload_c2(args, dev):
    import torch
    world, n, ch = 8, args.elems, args.channels
    full = n == 268_435_456 and ch == 4

    def make():
        if args.gpu_inputs:
            torch.manual_seed(0)
            return [torch.randn(n, device=dev, dtype=torch.float32).to(torch.bfloat16) for _ in range(world)]
        return headline_inputs(n, world, dev)

    def check(pristine, bufs):
        same = all(torch.equal(bufs[0].view(torch.int16), b.view(torch.int16)) for b in bufs[1:])
        want = ring_expected(pristine, n, ch)
        exact = torch.equal(want.view(torch.int16), bufs[0].view(torch.int16))
        ref32 = sum(p[:1 << 20].float() for p in pristine)
        rel = ((bufs[0][:1 << 20].float() - ref32).abs() / ref32.abs().clamp_min(1.0)).max().item()
        v = {"ranks_identical": bool(same), "matches_ring_order_bf16": bool(exact),
             "max_rel_err_vs_fp32_sum_first_1Mi": round(rel, 5), "output_sha256": sha256_of(bufs[0])}
        ok = same and exact
        golden_path = os.path.join(ROOT, "tests", "golden", "headline_sha256.json")
        if full and not args.gpu_inputs and os.path.exists(golden_path):
            golden = json.load(open(golden_path))
            v["input_rank0_matches_committed_sha256"] = sha256_of(pristine[0]) == golden["input_sha256_per_rank"][0]
            v["output_matches_committed_oracle_sha256"] = v["output_sha256"] == golden["output_sha256"]
            ok = ok and v["input_rank0_matches_committed_sha256"] and v["output_matches_committed_oracle_sha256"]
        return ok, v

    name = "ring_allreduce_sum_R8_bf16_512MiB_per_rank_4ch" if full else f"ring_allreduce_sum_R8_bf16_{n}elems_per_rank_{ch}ch"
    return Workload("c2", name, world, n, "bf16", graphs("ring", "build_allreduce", world, n, "bfloat16", ch), make, check,
                    "ring_allreduce_R8_bf16_512MiB" if full else None, ch)


def workload_c3(args, dev):
    import torch
    world, n = 16, 16_777_216

    def make():
        g = torch.Generator().manual_seed(0)
        return [(torch.rand(n, generator=g) * 2 - 1).to(dev) for _ in range(world)]

    def check(pristine, bufs):
        same = all(torch.equal(bufs[0].view(torch.int32), b.view(torch.int32)) for b in bufs[1:])
        # halving-doubling order: a balanced pairwise tree over the rank bits, low bit first
        vals = [p.clone() for p in pristine]
        k = 1
        while k < world:
            vals = [vals[r ^ k] + vals[r] if (r ^ k) > r else vals[r] + vals[r ^ k] for r in range(world)]
            k <<= 1
        exact = torch.equal(vals[0].view(torch.int32), bufs[0].view(torch.int32))
        ref = torch.stack([p.double() for p in pristine]).sum(0)
        rel = ((bufs[0].double() - ref).abs() / ref.abs().clamp_min(1.0)).max().item()
        return same and exact and rel < 1e-6 * world, {"ranks_identical": bool(same), "matches_pairwise_order_f32": bool(exact),
                                                     "max_rel_err_vs_f64_sum": float(f"{rel:.3g}"), "tolerance": 1e-6 * world}

    return Workload("c3", "rhd_allreduce_sum_R16_f32_64MiB_per_rank_2ch", world, n, "f32",
                    graphs("rhd", "build_allreduce", world, n, "float32", 2), make, check, "rhd_allreduce_R16_f32_64MiB", 2)


def workload_c5(args, dev):
    import torch
    from pccl_amd.dsl import ragged_cuts
    world, n = 32, 25_165_824
    cuts = ragged_cuts(n, 8, seed=0)
    is_int = args.c5_dtype == "int32"

    def make():
        g = torch.Generator().manual_seed(0)
        if is_int:
            return [torch.randint(-1000, 1000, (n,), generator=g, dtype=torch.int32).to(dev) for _ in range(world)]
        return [torch.randn(n, generator=g).to(dev) for _ in range(world)]

    def check(pristine, bufs):
        want = torch.stack(pristine).sum(0, dtype=torch.int32) if is_int else torch.stack(pristine).amax(0)
        ok = all(torch.equal(b.view(torch.int32), want.view(torch.int32)) for b in bufs)
        return ok, {"every_rank_equals_" + ("int32_wrapping_sum" if is_int else "f32_max"): bool(ok)}

    if is_int:
        return Workload("c5", "tree_allreduce_sum_R32_int32_96MiB_per_rank_ragged8", world, n, "int32",
                        graphs("tree", "build_allreduce", world, n, "int32", 1, reduce_op="sum", cuts=cuts), make, check,
                        "tree_allreduce_R32_int32_sum_96MiB")
    return Workload("c5", "tree_allreduce_max_R32_f32_96MiB_per_rank_ragged8", world, n, "f32",
                    graphs("tree", "build_allreduce", world, n, "float32", 1, reduce_op="max", cuts=cuts), make, check,
                    "tree_allreduce_R32_f32_max_96MiB")


# ----------------------------------------------------------------------------------------- helpers

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


def cpu_baseline(jsons, world: int, sample_elems: int, np_dtype: str, label: str, reps: int = 3):
    """Time the CPU oracle on the given graphs (`sample_elems` elements per rank)."""
    import numpy as np
    from oracle import oracle
    gs = [oracle.Graph(json.loads(j)) for j in jsons]
    rng = np.random.default_rng(0)
    threads = os.cpu_count() or 1
    env = os.environ.get("OMP_NUM_THREADS")
    if env and env.isdigit():
        threads = int(env)
    if np_dtype == "uint16":     # bf16 / f16 bit patterns of N(0,1)-like magnitudes; first touch by filling
        bufs = [rng.integers(0x3C00, 0x4000, sample_elems, dtype=np.uint16) for _ in range(world)]
    elif np_dtype == "int32":
        bufs = [rng.integers(-1000, 1000, sample_elems, dtype=np.int32) for _ in range(world)]
    else:
        bufs = [rng.standard_normal(sample_elems, dtype=np.float32) for _ in range(world)]
    stats = oracle.run(gs, bufs, threads=threads)      # warm-up
    times = []
    for _ in range(reps):
        t0 = time.perf_counter()
        stats = oracle.run(gs, bufs, threads=threads)
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
            "sample": f"{label} at {sample_elems} elements per rank, {stats.bytes} algorithmic bytes (every op moves its "
                      f"full bytes on the CPU), median of {reps} runs after 1 warm-up, {med * 1e3:.1f} ms"}


def kernel_source_sha256() -> str:
    """Hash of the kernel source the library was built from: a counter profile names the one it measured."""
    import hashlib
    with open(os.path.join(ROOT, "pccl_amd", "csrc", "kernels.hip"), "rb") as f:
        return hashlib.sha256(f.read()).hexdigest()


def committed_traffic(kernel: str, stem: str | None):
    """HBM bytes per launch from the committed rocprofv3 counter summary of `kernel` on the workload
    `stem` (FETCH_SIZE + WRITE_SIZE scaled by a 1 GiB copy), with the file it comes from.  The figure is
    only handed on while the profile was taken on the kernel source that is in the tree now (the file
    records its hash): after a kernel change `traffic` is null until the profile has been retaken."""
    if not stem:
        return None, None
    rel = os.path.join("profiles", f"{kernel}_{stem}.traffic.json")
    try:
        with open(os.path.join(ROOT, rel)) as f:
            rec = json.load(f)
    except (OSError, ValueError):
        return None, None
    if rec.get("kernels_hip_sha256") != kernel_source_sha256():
        return None, rel + " (taken on another version of kernels.hip: not used)"
    return rec.get("hbm_bytes_per_launch"), rel


def c4_traffic(kernel: str, kind: str, nbytes: int):
    """Counter-measured traffic of a staged reduce_scatter / allgather call: only the 512 MB size has a profile."""
    if nbytes != 536870912:
        return None, None
    return committed_traffic(kernel, f"ring_{kind}_R8_f16_512MB_staged")


def release_cached_memory() -> None:
    """Hands torch's cached blocks back to the driver.  Called where the next configuration uses
    tensors of other sizes, so that no configuration runs on pieces split off larger cached blocks
    (32 x 96 MiB carved out of cached 512 MiB blocks: 0.828 of peak against 0.842 on blocks of their
    own).  Where the next configuration uses the same sizes it takes the blocks over from the cache:
    memory that a process has freed to the driver and allocated again has been seen to be slower on
    this GPU (8 x 512 MB reduce_scatter, same process, same call: 0.808 of peak against 0.85 on the
    process's first allocations; not in every order of allocations).  PCCL_BENCH_FREE_TO_DRIVER=1
    releases after every configuration, for comparison."""
    import torch
    torch.cuda.empty_cache()


def release_between_equal_sizes() -> None:
    if os.environ.get("PCCL_BENCH_FREE_TO_DRIVER", "0") == "1":
        release_cached_memory()


def timed_inplace(eng, name, bufs, steps, warmup):
    """K timed executions in place: wall time per step and per-launch HIP-event times."""
    import torch
    for _ in range(warmup):
        eng.execute_inplace(name, bufs)
    torch.cuda.synchronize()
    ev0 = [torch.cuda.Event(enable_timing=True) for _ in range(steps)]
    ev1 = [torch.cuda.Event(enable_timing=True) for _ in range(steps)]
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(steps):
        ev0[i].record()
        eng.execute_inplace(name, bufs)
        ev1[i].record()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    return wall * 1e3 / steps, [a.elapsed_time(b) for a, b in zip(ev0, ev1)]


def moved_bytes(info: dict, mode: str, staged: bool = False):
    """HBM bytes one execution moves, by what kind of runner executes it."""
    if mode in ("stepwise", "persistent") or not info["position_aligned"]:
        return info["algorithmic_bytes"], "algorithmic bytes: every op moves its full bytes in this mode"
    if staged and info["staged_load_bytes"] + info["staged_store_bytes"] > 0:
        return info["staged_load_bytes"] + info["staged_store_bytes"], "bytes the column plan of the staged call loads and stores"
    return info["column_load_bytes"] + info["column_store_bytes"], "bytes the column plan loads and stores"


def reference_bandwidths(collective: str, data_bytes: int, world: int, ms_per_call: float) -> dict:
    """Per-rank bandwidths the reference's way (tests/bench_algo_comparison.py:141-156): alg_bw is the
    rank's full tensor (the allreduce tensor, the reduce_scatter input, the allgather output) over the
    time of one call, bus_bw scales it by 2 (N - 1) / N for an allreduce and (N - 1) / N otherwise."""
    alg = data_bytes / (ms_per_call * 1e-3) / 1e9
    factor = 2 * (world - 1) / world if collective == "allreduce" else (world - 1) / world
    return {"alg_bw_GBps": round(alg, 1), "bus_bw_GBps": round(alg * factor, 1),
            "bw_definition": "per virtual rank, reference tests/bench_algo_comparison.py:141-156"}


def side_leg(eng, name, bufs, mode, reps, alg_bytes):
    import torch
    eng.set_option("mode", mode)
    for _ in range(2):
        eng.execute_inplace(name, bufs)
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(reps):
        eng.execute_inplace(name, bufs)
    e1.record()
    torch.cuda.synchronize()
    ms = e0.elapsed_time(e1) / reps
    if mode == "persistent":
        eng.sync_operation(name)      # would raise if a bounded wait had expired
    eng.set_option("mode", "auto")
    rate = alg_bytes / (ms * 1e-3) / 1e9
    return {"mode": mode, "ms_per_step": round(ms, 4), "GB/s": round(rate, 1), "frac_of_hbm_peak": round(rate / PEAK_GBPS, 4),
            "note": "HBM traffic equals the algorithmic bytes in this mode: every op moves its full bytes"}


# ----------------------------------------------------------------------------------------- in-place configurations

def run_inplace(args, wl: Workload, dev) -> int:
    import torch
    from pccl_amd.engine import Engine
    eng = Engine(wl.world, 0)
    for r, text in enumerate(wl.jsons):
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
    runner_kernel = eng.get_option("runner_inplace:bench")      # the kernel the library launches for this plan, size and options
    log(f"program: {info}; runner: {runner_kernel}")

    t0 = time.perf_counter()
    pristine = wl.make_inputs()
    log(f"inputs generated in {time.perf_counter() - t0:.1f} s")
    if args.rank_skew_bytes:
        # rank buffers carved out of one allocation, rank r starting r * (size + skew) bytes in: the same
        # position of different ranks then falls on different memory channels
        es = pristine[0].element_size()
        stride = wl.n + args.rank_skew_bytes // es
        arena = torch.empty(wl.world * stride, dtype=pristine[0].dtype, device=dev)
        bufs = [arena[r * stride:r * stride + wl.n] for r in range(wl.world)]
        for b, p in zip(bufs, pristine):
            b.copy_(p)
    else:
        bufs = [p.clone() for p in pristine]
    log("rank buffer addresses: " + " ".join(hex(b.data_ptr()) for b in bufs[:4]) + " ...")

    # the first execution in the process (tables just uploaded, nothing of the buffers in any cache)
    c0, c1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    c0.record()
    eng.execute_inplace("bench", bufs)
    c1.record()
    torch.cuda.synchronize()
    cold_ms = c0.elapsed_time(c1)

    verify = {}
    if not args.no_verify:
        ok, verify = wl.check(pristine, bufs)
        log(f"verify: {verify}")
        if not ok:
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

    ms_per_step, kern_ms = timed_inplace(eng, "bench", bufs, args.steps, args.warmup)
    avg_ms = sum(kern_ms) / len(kern_ms)
    hbm_bytes, hbm_note = moved_bytes(info, args.mode)
    value = hbm_bytes / (ms_per_step * 1e-3) / 1e9
    achieved = hbm_bytes / (avg_ms * 1e-3) / 1e9
    reps = max(3, args.steps // 4)

    # end to end the reference's way: input and output staging copies included
    staged = None
    if wl.key == "c2":
        outs = [torch.empty_like(p) for p in pristine]
        eng.execute_operation("bench", pristine, outs)
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(reps):
            eng.execute_operation_async("bench", pristine, outs)
        e1.record()
        torch.cuda.synchronize()
        staged_ms = e0.elapsed_time(e1) / reps
        del outs
        sb, _ = moved_bytes(info, args.mode, staged=True)
        staged = {"ms_per_call": round(staged_ms, 4), "hbm_GB/s": round(sb / (staged_ms * 1e-3) / 1e9, 1),
                  **reference_bandwidths("allreduce", wl.n * 2, wl.world, staged_ms),
                  "note": "the reference's call shape (separate input and output tensors per rank, execute_operation_async); "
                          "in column mode the staging copies are fused into the program, so this is again one launch"}

    # the same graph op by op (one launch per dependency level), and as one persistent launch whose
    # workgroups order themselves through device-side flags
    op_by_op = persistent = None
    if args.mode == "auto" and not args.no_side_legs:
        op_by_op = side_leg(eng, "bench", bufs, "stepwise", reps, alg_bytes)
        persistent = side_leg(eng, "bench", bufs, "persistent", reps, alg_bytes)
        persistent["note"] += "; one launch for the whole graph, ordering by device-side flags (one per work item, one ready word per op)"

    default_runner = not any(kv.split("=")[0].startswith(("lds_slots", "slot_", "phased")) for kv in args.option)
    kernel = runner_kernel
    traffic, traffic_source = committed_traffic(kernel, wl.traffic_stem) if default_runner else (None, None)
    if traffic is not None and kernel == "level_kernel":
        traffic *= info["num_levels"]      # the profile gives one launch; an execution is one launch per level
    result = {
        "metric": METRIC + ", " + ("8-vrank 512MB bf16 ring allreduce graph" if wl.key == "c2" else wl.name),
        "value": round(value, 1), "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": wl.dtype, "data": "synthetic",
        "config": {"workload": wl.name, "virtual_ranks": wl.world, "bytes_per_rank": wl.n * (2 if wl.dtype in ("bf16", "f16") else 4),
                   "channels": wl.channels, "data_ops": info["num_data_ops"], "algorithmic_bytes_per_step": alg_bytes,
                   "hbm_bytes_per_step": hbm_bytes, "mode": args.mode, "in_place": True},
        "pct_of_hbm_peak": round(100 * value / PEAK_GBPS, 1),
        "algorithmic_equiv_GBps": round(alg_bytes / (ms_per_step * 1e-3) / 1e9, 1),
        **reference_bandwidths("allreduce", wl.n * (2 if wl.dtype in ("bf16", "f16") else 4), wl.world, ms_per_step),
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": PEAK_GBPS, "unit": "GB/s",
                     "frac": round(achieved / PEAK_GBPS, 4), "traffic": traffic, "traffic_source": traffic_source,
                     "bytes_counted": hbm_note, "kernel": kernel,
                     "kernel_ms_avg": round(avg_ms, 4), "kernel_ms_min": round(min(kern_ms), 4),
                     "kernel_ms_median": round(sorted(kern_ms)[len(kern_ms) // 2], 4),
                     "kernel_ms_first_execution": round(cold_ms, 4),
                     "planned_load_bytes": info["column_load_bytes"], "planned_store_bytes": info["column_store_bytes"]},
        "end_to_end_staged": staged,
        "op_by_op": op_by_op,
        "single_launch_flag_ordered": persistent,
        "device": device_info(dev),
        "verify": verify,
    }
    if traffic:
        result["roofline"]["traffic_vs_counted"] = round(traffic / hbm_bytes, 4)
    if args.gpu_inputs:
        result["data"] = "synthetic (GPU generator: tuning run)"
    del bufs, pristine
    eng.close()
    release_between_equal_sizes()     # the 512 MB pair of configuration 4 comes next, on blocks of the same size
    if not args.no_cpu_baseline:
        np_dtype = "uint16" if wl.dtype in ("bf16", "f16") else "int32" if wl.dtype == "int32" else "float32"
        result["cpu_baseline"] = cpu_baseline(wl.jsons, wl.world, wl.n, np_dtype, wl.name + ": the same graphs", args.cpu_reps)
    # the other configurations, after everything of the headline has been measured
    full_default = (wl.key == "c2" and args.mode == "auto" and default_runner and not args.gpu_inputs
                    and args.elems == 268_435_456 and args.channels == 4 and args.num_blocks < 0 and not args.rank_skew_bytes)
    if args.other_configs == "on" or (args.other_configs == "auto" and full_default and not args.no_side_legs):
        result["other_configs"] = other_configs(args, dev)
        if not all(row["verified"] for row in result["other_configs"]):
            print(json.dumps({"error": "verification of another configuration failed",
                              "other_configs": result["other_configs"]}))
            return 1
    print(json.dumps(result))
    return 0


# ----------------------------------------------------------------------------------------- the other configurations, briefly

def brief_inplace(args, wl: Workload, dev) -> dict:
    """One of the other in-place configurations inside the default run: first execution verified at
    full size as in its own run, then `steps` timed executions with HIP events."""
    import torch
    from pccl_amd.engine import Engine
    eng = Engine(wl.world, 0)
    try:
        for r, text in enumerate(wl.jsons):
            eng.register_operation_json("bench", text, r)
        info = eng.op_info("bench")
        pristine = wl.make_inputs()
        bufs = [p.clone() for p in pristine]
        eng.execute_inplace("bench", bufs)
        torch.cuda.synchronize()
        ok, verify = wl.check(pristine, bufs)
        for b, p in zip(bufs, pristine):
            b.copy_(p)
        ms_per_step, kern_ms = timed_inplace(eng, "bench", bufs, args.steps, args.warmup)
        avg_ms = sum(kern_ms) / len(kern_ms)
        hbm_bytes, note = moved_bytes(info, "auto")
        rate = hbm_bytes / (avg_ms * 1e-3) / 1e9
        kernel = eng.get_option("runner_inplace:bench")
        traffic, source = committed_traffic(kernel, wl.traffic_stem)
        out = {"workload": wl.name, "kernel": kernel, "verified": bool(ok), "verify": verify, "ms_per_step": round(ms_per_step, 4),
               "kernel_ms_avg": round(avg_ms, 4), "kernel_ms_min": round(min(kern_ms), 4),
               "hbm_bytes_per_step": hbm_bytes, "algorithmic_bytes_per_step": info["algorithmic_bytes"],
               "GB/s": round(rate, 1), "frac": round(rate / PEAK_GBPS, 4), "bytes_counted": note,
               "traffic": traffic, "traffic_source": source}
        out.update(reference_bandwidths("allreduce", wl.n * (2 if wl.dtype in ("bf16", "f16") else 4), wl.world, ms_per_step))
        return out
    finally:
        eng.close()


def brief_c4(args, dev, nbytes: int) -> list:
    """The 512 MB end point of configuration 4 inside the default run: ring reduce_scatter and
    allgather, 8 ranks, fp16, as staged calls on separate input and output tensors; the first call is
    verified against the ring's reduction order evaluated with torch's fp16 adds."""
    import torch
    from pccl_amd.engine import Engine
    world, n = 8, nbytes // 2
    chunk = n // world
    g = torch.Generator(device="cuda").manual_seed(0)
    out = []
    for method, in_elems, out_elems in (("build_reduce_scatter", n, chunk), ("build_allgather", chunk, n)):
        eng = Engine(world, 0)
        try:
            for r, j in enumerate(graphs("ring", method, world, n, "float16", 1)):
                eng.register_operation_json("bench", j, r)
            info = eng.op_info("bench")
            x = [(torch.randn(in_elems, generator=g, device="cuda") * 0.1).half() for _ in range(world)]
            outs = [torch.empty(out_elems, dtype=torch.float16, device="cuda") for _ in range(world)]
            call = eng.prepare("bench", x, outs)
            call()
            torch.cuda.synchronize()
            ok = True
            if method == "build_reduce_scatter":
                for c in range(world):          # chunk c: x_(c+1), then + x_(c+2) ... + x_c, each sum rounded to fp16
                    acc = x[(c + 1) % world][c * chunk:(c + 1) * chunk].clone()
                    for k in range(2, world + 1):
                        acc = acc + x[(c + k) % world][c * chunk:(c + 1) * chunk]
                    ok = ok and torch.equal(acc.view(torch.int16), outs[c].view(torch.int16))
            else:
                whole = torch.cat(x)
                ok = all(torch.equal(o.view(torch.int16), whole.view(torch.int16)) for o in outs)
                del whole
            for _ in range(args.warmup):
                call()
            torch.cuda.synchronize()
            ev = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(args.steps)]
            t0 = time.perf_counter()
            for a, b in ev:
                a.record()
                call()
                b.record()
            torch.cuda.synchronize()
            wall_ms = (time.perf_counter() - t0) * 1e3 / args.steps
            ms = [a.elapsed_time(b) for a, b in ev]
            avg = sum(ms) / len(ms)
            hbm, note = moved_bytes(info, "auto", staged=True)
            rate = hbm / (avg * 1e-3) / 1e9
            kind = method[6:]
            row = {"workload": f"ring_{kind}_R8_f16_{nbytes}B_per_rank_staged_call", "kernel": eng.get_option("runner_staged:bench"), "verified": bool(ok),
                   "verify": {"matches_ring_order_f16" if kind == "reduce_scatter" else "every_output_is_the_concatenation": bool(ok)},
                   "ms_per_step": round(wall_ms, 4), "kernel_ms_avg": round(avg, 4), "kernel_ms_min": round(min(ms), 4),
                   "hbm_bytes_per_step": hbm, "algorithmic_bytes_per_step": info["algorithmic_bytes"],
                   "GB/s": round(rate, 1), "frac": round(rate / PEAK_GBPS, 4), "bytes_counted": note}
            row["traffic"], row["traffic_source"] = c4_traffic(row["kernel"], kind, nbytes)
            row.update(reference_bandwidths(kind, nbytes, world, wall_ms))
            out.append(row)
        finally:
            eng.close()
            del x, outs
            release_between_equal_sizes()     # the allgather's tensors have the reduce_scatter's sizes, swapped
    return out


def other_configs(args, dev) -> list:
    """Configurations 3, 5 (both element types) and the 512 MB pair of 4, each verified and timed like
    its own `--config` run, for the default run's JSON line."""
    saved = args.c5_dtype
    try:
        # the 512 MB pair first: its tensors have the size of the headline's, whose blocks it takes over
        c4 = brief_c4(args, dev, 512 << 20)
        release_cached_memory()
        rows = [brief_inplace(args, workload_c3(args, dev), dev)]
        release_cached_memory()
        for dt in ("int32", "float32"):
            args.c5_dtype = dt
            rows.append(brief_inplace(args, workload_c5(args, dev), dev))
            release_between_equal_sizes()
        release_cached_memory()
        rows.extend(c4)
    finally:
        args.c5_dtype = saved
    return rows


# ----------------------------------------------------------------------------------------- c4: message-size sweep

def run_c4(args, dev) -> int:
    """Ring reduce_scatter and allgather, 8 ranks, fp16, N(0, 0.1) inputs, 4 KB to 512 MB per rank,
    as staged calls (the reference's call shape: separate input and output tensors).  One JSON line
    per collective and size: latency per call and HBM rate; the knee is the result."""
    import torch
    from pccl_amd.engine import Engine
    world = 8
    sizes = [4096 * 4 ** k for k in range(9)] + [512 << 20]
    if args.c4_bytes:
        sizes = [int(s) for s in args.c4_bytes.split(",")]
    g = torch.Generator(device="cuda").manual_seed(0)
    if args.calibrate_copy_bytes:
        from pccl_amd import _lib
        src = torch.empty(args.calibrate_copy_bytes, dtype=torch.uint8, device=dev).random_(0, 256)
        dst = torch.empty_like(src)
        for _ in range(3):
            _lib.check(_lib.lib().pccl_hip_copy(3, src.data_ptr(), dst.data_ptr(), src.numel(), None))
        torch.cuda.synchronize()
        del src, dst
    for nbytes in sizes:
        n = nbytes // 2
        chunk = n // world
        for method, in_elems, out_elems in (("build_reduce_scatter", n, chunk), ("build_allgather", chunk, n)):
            eng = Engine(world, 0)
            try:
                jsons = graphs("ring", method, world, n, "float16", 1)
                for r, j in enumerate(jsons):
                    eng.register_operation_json("bench", j, r)
                eng.set_option("mode", args.mode)
                for kv in args.option:
                    key, _, val = kv.partition("=")
                    eng.set_option(key, val)
                info = eng.op_info("bench")
                x = [(torch.randn(in_elems, generator=g, device="cuda") * 0.1).half() for _ in range(world)]
                outs = [torch.empty(out_elems, dtype=torch.float16, device="cuda") for _ in range(world)]
                call = eng.prepare("bench", x, outs)
                for _ in range(args.warmup):
                    call()
                torch.cuda.synchronize()
                if args.c4_graph:
                    # the prepared call recorded once into a graph (one kernel node in column mode) and replayed
                    side = torch.cuda.Stream()
                    side.wait_stream(torch.cuda.current_stream())
                    graph = torch.cuda.CUDAGraph()
                    with torch.cuda.stream(side):
                        with torch.cuda.graph(graph, stream=side):
                            call()
                    torch.cuda.current_stream().wait_stream(side)
                    call = graph.replay
                    for _ in range(args.warmup):
                        call()
                    torch.cuda.synchronize()
                ev = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(args.steps)]
                t0 = time.perf_counter()
                for a, b in ev:
                    a.record()
                    call()
                    b.record()
                torch.cuda.synchronize()
                wall_ms = (time.perf_counter() - t0) * 1e3 / args.steps
                ms = sorted(a.elapsed_time(b) for a, b in ev)
                avg = sum(ms) / len(ms)
                hbm, note = moved_bytes(info, args.mode, staged=True)
                c4_kernel = eng.get_option("runner_staged:bench")
                c4_tr = c4_traffic(c4_kernel, method[6:], nbytes) if args.mode == "auto" and not args.option else (None, None)
                if args.mode in ("stepwise", "persistent"):
                    hbm += 2 * 2 * world * (in_elems + out_elems)  # the two batched staging copies: read + write, 2 bytes per element
                    note += " plus the input and output staging copies"
                print(json.dumps({
                    "metric": METRIC + f", ring {method[6:]} R8 fp16 staged call", "value": round(hbm / (wall_ms * 1e-3) / 1e9, 1), "unit": "GB/s",
                    "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(wall_ms, 4), "higher_is_better": True,
                    "scaling": "weak", "vs_baseline": None, "dtype": "f16", "data": "synthetic",
                    "config": {"workload": f"ring_{method[6:]}_R8_f16_{nbytes}B_per_rank", "virtual_ranks": world, "bytes_per_rank": nbytes,
                               "channels": 1, "data_ops": info["num_data_ops"], "algorithmic_bytes_per_step": info["algorithmic_bytes"],
                               "hbm_bytes_per_step": hbm, "mode": args.mode, "in_place": False, "graph_replay": bool(args.c4_graph)},
                    "wall_us_per_call": round(wall_ms * 1e3, 2),
                    "latency_us_median": round(ms[len(ms) // 2] * 1e3, 2), "latency_us_min": round(ms[0] * 1e3, 2),
                    **reference_bandwidths(method[6:], nbytes, world, wall_ms),
                    "algorithmic_equiv_GBps": round(info["algorithmic_bytes"] / (wall_ms * 1e-3) / 1e9, 1),
                    "roofline": {"bound": "hbm", "achieved": round(hbm / (avg * 1e-3) / 1e9, 1), "peak": PEAK_GBPS, "unit": "GB/s",
                                 "frac": round(hbm / (avg * 1e-3) / 1e9 / PEAK_GBPS, 4), **dict(zip(("traffic", "traffic_source"), c4_tr)),
                                 "kernel": c4_kernel, "bytes_counted": note, "kernel_ms_avg": round(avg, 5)}}), flush=True)
            finally:
                eng.close()
    return 0


# ----------------------------------------------------------------------------------------- main

def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--config", default="c2", choices=["c2", "c3", "c4", "c5"])
    ap.add_argument("--mode", default="auto")
    ap.add_argument("--elems", type=int, default=268_435_456, help="c2: elements per rank (default: the headline size)")
    ap.add_argument("--channels", type=int, default=4, help="c2: channels of the ring")
    ap.add_argument("--c5-dtype", default="int32", choices=["int32", "float32"], help="c5: int32 SUM or float32 MAX")
    ap.add_argument("--c4-bytes", default="", help="c4: comma-separated bytes per rank instead of the full sweep")
    ap.add_argument("--c4-graph", action="store_true", help="c4: record the prepared call into a HIP graph once and time its replays")
    ap.add_argument("--vecs-per-thread", type=int, default=0)
    ap.add_argument("--num-blocks", type=int, default=-1)
    ap.add_argument("--option", action="append", default=[], metavar="KEY=VALUE",
                    help="engine option to set before the run (e.g. lds_slots=0, slot_threads=128); repeatable")
    ap.add_argument("--rank-skew-bytes", type=int, default=0,
                    help="carve the rank buffers out of one allocation, each this many bytes further in than its size")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-verify", action="store_true")
    ap.add_argument("--no-side-legs", action="store_true", help="skip the op-by-op and single-launch legs of an auto-mode run")
    ap.add_argument("--gpu-inputs", action="store_true",
                    help="c2: draw the inputs with the GPU generator (tuning runs only; not the prescribed inputs)")
    ap.add_argument("--other-configs", default="auto", choices=["auto", "on", "off"],
                    help="append configurations 3, 5 and the 512 MB pair of 4 (verified, timed) to the JSON line as "
                         "'other_configs': auto = only in the plain default run")
    ap.add_argument("--cpu-reps", type=int, default=20)
    ap.add_argument("--calibrate-copy-bytes", type=int, default=0,
                    help="also launch the library's plain copy kernel on this many bytes (3 times): a "
                         "known-traffic reference for scaling rocprofv3 FETCH_SIZE / WRITE_SIZE")
    ap.add_argument("--probe", default="", metavar="'RANKS BYTES CASE ...'",
                    help="run the memory-system probe (pccl_amd/csrc/stream_probe.hip: bare kernels of the runners' traffic "
                         "shapes) with these arguments instead of a benchmark; prints its JSON lines")
    args = ap.parse_args()
    if args.probe:
        # a child process, started before anything here touches the GPU
        import subprocess
        from pccl_amd import build as lib_build
        if not os.path.exists(lib_build.PROBE):
            print("bench.py: the probe is not built (python pccl_amd/build.py)", file=sys.stderr)
            return 1
        return subprocess.run([lib_build.PROBE] + args.probe.split()).returncode
    if args.gpus != 1:
        print("bench.py: this build runs on one GPU: the R ranks are virtual ranks resident in one "
              "MI355X's HBM and no multi-GPU path exists; run with --gpus 1", file=sys.stderr)
        return 2

    import torch
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible; the executor has no CPU fallback", file=sys.stderr)
        return 1
    dev = torch.device("cuda", 0)
    if args.config == "c4":
        return run_c4(args, dev)
    wl = {"c2": workload_c2, "c3": workload_c3, "c5": workload_c5}[args.config](args, dev)
    return run_inplace(args, wl, dev)


if __name__ == "__main__":
    sys.exit(main())
