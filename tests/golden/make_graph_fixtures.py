"""Regenerate tests/golden/graphs/*.json from the reference DSL (run in the authoring container only).

The reference package cannot be imported whole here: ``pccl/__init__`` pulls in the superoptimizer,
which needs ``z3`` (not installed), and ``pccl.engine`` needs the compiled CUDA extension.  The
schedule templates and the JSON generator depend on neither, so this script loads exactly those
modules (``nodes``, ``graph``, ``decorators``, ``passes.{dependency_analysis,dce}``,
``codegen.{mapping,json_generator}``, ``algorithms.{base,ring,recursive_hd,tree}``) under a synthetic package skeleton and writes the JSON v2 text the reference
emits for a handful of small configurations.  The fixtures are data (compiler output), not source.

Usage:  python tests/golden/make_graph_fixtures.py [/root/reference]
"""
import importlib.util
import json
import os
import sys
import types

REF = sys.argv[1] if len(sys.argv) > 1 else "/root/reference"
OUT = os.path.join(os.path.dirname(os.path.abspath(__file__)), "graphs")


def _pkg(name, path):
    m = types.ModuleType(name)
    m.__path__ = [path]
    m.__package__ = name
    sys.modules[name] = m
    return m


def _load(name, relpath):
    spec = importlib.util.spec_from_file_location(name, os.path.join(REF, relpath))
    m = importlib.util.module_from_spec(spec)
    sys.modules[name] = m
    spec.loader.exec_module(m)
    return m


def load_reference_dsl():
    _pkg("pccl", os.path.join(REF, "pccl"))
    _pkg("pccl.dsl", os.path.join(REF, "pccl/dsl"))
    _pkg("pccl.dsl.algorithms", os.path.join(REF, "pccl/dsl/algorithms"))
    _load("pccl.dsl.nodes", "pccl/dsl/nodes.py")
    _load("pccl.dsl.graph", "pccl/dsl/graph.py")
    _load("pccl.dsl.decorators", "pccl/dsl/decorators.py")
    # ``passes/__init__`` and ``compiler.py`` import the channelize pass, which imports the
    # superoptimizer (z3).  The default pipeline of ``compile_to_json_string`` never runs that pass
    # (enable_channelize=False, enable_superopt=False): it is DependencyAnalysis -> DCE ->
    # DependencyAnalysis -> RuntimeGraphGenerator (pccl/dsl/compiler.py:33-54,67-69), so those
    # three reference classes are loaded directly and driven in that order below.
    _pkg("pccl.dsl.passes", os.path.join(REF, "pccl/dsl/passes"))
    _pkg("pccl.dsl.codegen", os.path.join(REF, "pccl/dsl/codegen"))
    dep = _load("pccl.dsl.passes.dependency_analysis", "pccl/dsl/passes/dependency_analysis.py")
    dce = _load("pccl.dsl.passes.dce", "pccl/dsl/passes/dce.py")
    _load("pccl.dsl.codegen.mapping", "pccl/dsl/codegen/mapping.py")
    gen = _load("pccl.dsl.codegen.json_generator", "pccl/dsl/codegen/json_generator.py")

    def compile_to_json_string(graph):
        dep.DependencyAnalysisPass().run(graph)
        dce.DeadCodeEliminationPass().run(graph)
        dep.DependencyAnalysisPass().run(graph)
        return gen.RuntimeGraphGenerator(indent=2).generate_string(graph)

    comp = types.SimpleNamespace(compile_to_json_string=compile_to_json_string)
    _load("pccl.dsl.algorithms.base", "pccl/dsl/algorithms/base.py")
    ring = _load("pccl.dsl.algorithms.ring", "pccl/dsl/algorithms/ring.py")
    rhd = _load("pccl.dsl.algorithms.recursive_hd", "pccl/dsl/algorithms/recursive_hd.py")
    tree = _load("pccl.dsl.algorithms.tree", "pccl/dsl/algorithms/tree.py")
    pipe = _load("pccl.dsl.pipeline", "pccl/dsl/pipeline.py")
    # the channelize pass and the cost model it consults: plain Python, loaded without running
    # superopt/__init__ (which needs z3)
    _pkg("pccl.dsl.superopt", os.path.join(REF, "pccl/dsl/superopt"))
    _load("pccl.dsl.superopt.rule", "pccl/dsl/superopt/rule.py")
    _load("pccl.dsl.superopt.cost_model", "pccl/dsl/superopt/cost_model.py")
    chan = _load("pccl.dsl.passes.channelize", "pccl/dsl/passes/channelize.py")

    def compile_channelized(graph, num_channels):
        dep.DependencyAnalysisPass().run(graph)
        dce.DeadCodeEliminationPass().run(graph)
        chan.ChannelizePass(num_channels=num_channels).run(graph)
        dep.DependencyAnalysisPass().run(graph)
        return gen.RuntimeGraphGenerator(indent=2).generate_string(graph)

    comp.compile_channelized = compile_channelized
    comp.decorators = sys.modules["pccl.dsl.decorators"]
    comp.Pipeline = pipe.Pipeline
    return comp, ring, rhd, tree


def pipelined_ring_allreduce(CommunicationOp, Pipeline, rank, world, n, dtype, depth):
    """Ring allreduce whose steps rotate over `depth` channels through the Pipeline construct; every
    notify / wait pair has its own signal id.  The schedule is the one the reference's bandwidth
    script builds (tests/bench_allreduce_tma_bw.py:119-186); tests/test_emitter.py holds the same
    function over the package under test."""
    chunk = n // world
    prev_rank, next_rank = (rank - 1) % world, (rank + 1) % world
    with CommunicationOp(name=f"ar_pipe{depth}_rank{rank}") as op:
        op.tensor(dtype=dtype, shape=(n,))
        pipe = Pipeline(depth=depth)
        sig = 0
        with pipe.bind(op):
            for _ in range(depth):
                with pipe.stage():
                    sig += 1
                    op.notify(signal_id=sig, target_rank=next_rank)
                    op.wait_notify(signal_id=sig, source_rank=prev_rank)
            for step in range(world - 1):
                with pipe.stage():
                    off = ((rank - step - 1) % world) * chunk
                    if step > 0:
                        sig += 1
                        op.wait_notify(signal_id=sig, source_rank=prev_rank)
                    op.sm_reduce(reduce_op="sum", source_rank=prev_rank, src_offset=off, dst_offset=off,
                                 remote_offset=off, count=chunk)
                    sig += 1
                    op.notify(signal_id=sig, target_rank=next_rank)
            for step in range(world - 1):
                with pipe.stage():
                    off = ((rank - step) % world) * chunk
                    sig += 1
                    op.wait_notify(signal_id=sig, source_rank=prev_rank)
                    op.sm_copy(source_rank=prev_rank, src_offset=off, dst_offset=off, size=chunk)
                    sig += 1
                    op.notify(signal_id=sig, target_rank=next_rank)
            for _ in range(depth):
                with pipe.stage():
                    sig += 1
                    op.wait_notify(signal_id=sig, source_rank=prev_rank)
        return op.get_graph()


def chained_gather(CommunicationOp, rank, world, chunk, dtype, pieces, kind):
    """A chain that the channelize pass accepts: `pieces` same-type data ops from the next rank whose
    source ranges follow one another, a notify / wait pair between every two, closed by a notify.
    tests/helpers.py holds the same function over the package under test."""
    peer = (rank + 1) % world
    with CommunicationOp(name=f"chain_{kind}_rank{rank}") as op:
        op.tensor(dtype=dtype, shape=(pieces * chunk,))
        op.notify(signal_id=1, target_rank=(rank - 1) % world)
        op.wait_notify(signal_id=1, source_rank=peer)
        for k in range(pieces):
            if kind == "copy":
                op.sm_copy(source_rank=peer, src_offset=k * chunk, dst_offset=k * chunk, size=chunk)
            else:
                op.tma_reduce(reduce_op="sum", source_rank=peer, src_offset=k * chunk, dst_offset=k * chunk,
                              remote_offset=k * chunk, count=chunk)
            if k % 2 == 1:
                op.notify(signal_id=10 + k, target_rank=(rank - 1) % world)
                op.wait_notify(signal_id=10 + k, source_rank=peer)
        op.notify(signal_id=2, target_rank=(rank - 1) % world)
        op.wait_notify(signal_id=2, source_rank=peer)
        return op.get_graph()


CHANNELIZE_CASES = [
    # (file stem, world, chunk, dtype, pieces, kind, num_channels)
    ("chan_copy_w2_c65536_f32_p8_nc2", 2, 65536, "float32", 8, "copy", 2),
    ("chan_reduce_w2_c16384_bf16_p7_nc3", 2, 16384, "bfloat16", 7, "reduce", 3),
    ("chan_copy_w2_c256_f16_p6_nc2", 2, 256, "float16", 6, "copy", 2),       # below min_data_size: untouched
    ("chan_copy_w2_c65536_f32_p2_nc2", 2, 65536, "float32", 2, "copy", 2),   # chain not longer than channels
]


PIPELINE_CASES = [
    # (file stem, world, tensor_size, dtype, depth)
    ("pipe_ring_ar_w4_n4096_bf16_d2", 4, 4096, "bfloat16", 2),
    ("pipe_ring_ar_w3_n3072_f32_d3", 3, 3072, "float32", 3),
]


CASES = [
    # (file stem, algorithm, method, world, tensor_size, dtype, executor, channels)
    ("ring_ar_sm_w2_n2048_bf16_c1", "ring", "build_allreduce", 2, 2048, "bfloat16", "sm", 1),
    ("ring_ar_sm_w4_n4096_f32_c2", "ring", "build_allreduce", 4, 4096, "float32", "sm", 2),
    ("ring_ar_tma_w8_n8192_bf16_c4", "ring", "build_allreduce", 8, 8192, "bfloat16", "tma", 4),
    ("ring_rs_sm_w4_n4096_f16_c1", "ring", "build_reduce_scatter", 4, 4096, "float16", "sm", 1),
    ("ring_ag_sm_w4_n4096_f16_c1", "ring", "build_allgather", 4, 4096, "float16", "sm", 1),
    ("ring_a2a_sm_w4_n4096_bf16_c1", "ring", "build_alltoall", 4, 4096, "bfloat16", "sm", 1),
    ("rhd_ar_sm_w8_n4096_f32_c1", "rhd", "build_allreduce", 8, 4096, "float32", "sm", 1),
    ("rhd_ar_tma_w4_n1024_bf16_c1", "rhd", "build_allreduce", 4, 1024, "bfloat16", "tma", 1),
    ("tree_ar_sm_w8_n1024_f32_c1", "tree", "build_allreduce", 8, 1024, "float32", "sm", 1),
    ("tree_ar_tma_w4_n512_f16_c1", "tree", "build_allreduce", 4, 512, "float16", "tma", 1),
]


def main():
    comp, ring, rhd, tree = load_reference_dsl()
    algs = {"ring": ring.RingAllreduce, "rhd": rhd.RecursiveHalvingDoubling,
            "tree": tree.TreeAllreduce}
    os.makedirs(OUT, exist_ok=True)
    index = []
    for stem, alg, method, world, n, dtype, executor, ch in CASES:
        for rank in range(world):
            g = getattr(algs[alg](), method)(rank, world, n, dtype=dtype, executor=executor,
                                             num_channels=ch)
            text = comp.compile_to_json_string(g)
            # compact re-serialisation keeps key order and values, drops the indent whitespace
            doc = json.loads(text)
            path = os.path.join(OUT, f"{stem}_rank{rank}.json")
            with open(path, "w") as f:
                json.dump(doc, f, separators=(",", ":"))
                f.write("\n")
        index.append({"stem": stem, "algorithm": alg, "method": method, "world_size": world,
                      "tensor_size": n, "dtype": dtype, "executor": executor,
                      "num_channels": ch})
    for stem, world, n, dtype, depth in PIPELINE_CASES:
        for rank in range(world):
            g = pipelined_ring_allreduce(comp.decorators.CommunicationOp, comp.Pipeline, rank, world, n, dtype, depth)
            doc = json.loads(comp.compile_to_json_string(g))
            with open(os.path.join(OUT, f"{stem}_rank{rank}.json"), "w") as f:
                json.dump(doc, f, separators=(",", ":"))
                f.write("\n")
        index.append({"stem": stem, "algorithm": "pipelined_ring", "method": "build_allreduce", "world_size": world,
                      "tensor_size": n, "dtype": dtype, "executor": "sm", "num_channels": depth})
    for stem, world, chunk, dtype, pieces, kind, nc in CHANNELIZE_CASES:
        for rank in range(world):
            g = chained_gather(comp.decorators.CommunicationOp, rank, world, chunk, dtype, pieces, kind)
            doc = json.loads(comp.compile_channelized(g, nc))
            with open(os.path.join(OUT, f"{stem}_rank{rank}.json"), "w") as f:
                json.dump(doc, f, separators=(",", ":"))
                f.write("\n")
        index.append({"stem": stem, "algorithm": "chained_gather", "method": kind, "world_size": world,
                      "tensor_size": pieces * chunk, "dtype": dtype, "executor": "sm" if kind == "copy" else "tma",
                      "num_channels": nc, "pieces": pieces})
    with open(os.path.join(OUT, "index.json"), "w") as f:
        json.dump(index, f, indent=1)
        f.write("\n")
    print(f"wrote {sum(c[3] for c in CASES) + sum(c[1] for c in PIPELINE_CASES) + sum(c[1] for c in CHANNELIZE_CASES)} graphs to {OUT}")


if __name__ == "__main__":
    main()
