"""Writes tests/golden/headline_sha256.json: sha256 of every rank's input of the headline workload
(8 ranks x 268,435,456 bf16, torch CPU generator seed 0, 8 slices per rank) and of the result the
CPU oracle computes for the 4-channel ring allreduce graph on them.  bench.py checks the GPU's
result against the output hash at full size.  Needs about 5 GiB of host memory and a minute.

    python tests/golden/make_headline_sha256.py
"""
import hashlib
import json
import os
import sys

import numpy as np
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
from oracle import oracle  # noqa: E402
from pccl_amd.dsl import RingAllreduce, compile_to_json_string  # noqa: E402

R, N, CHANNELS, SLICES = 8, 268_435_456, 4, 8


def main() -> int:
    g = torch.Generator().manual_seed(0)
    per = N // SLICES
    bufs, shas = [], []
    for r in range(R):
        raw = np.empty(N, dtype=np.uint16)
        for s in range(SLICES):
            raw[s * per:(s + 1) * per] = torch.randn(per, generator=g).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
        shas.append(hashlib.sha256(raw.tobytes()).hexdigest())
        bufs.append(raw)
        print(f"rank {r} input {shas[-1]}", flush=True)
    graphs = [oracle.Graph(json.loads(compile_to_json_string(
        RingAllreduce().build_allreduce(r, R, N, dtype="bfloat16", executor="sm", num_channels=CHANNELS)))) for r in range(R)]
    oracle.run(graphs, bufs)
    outs = [hashlib.sha256(b.tobytes()).hexdigest() for b in bufs]
    assert len(set(outs)) == 1, "the ranks disagree"
    print("output", outs[0], flush=True)
    doc = {"workload": "ring_allreduce_sum_R8_bf16_512MiB_per_rank_4ch",
           "input_rule": "torch.Generator().manual_seed(0); for rank 0..7, for slice 0..7: "
                         "torch.randn(33554432, generator=g).to(bfloat16); a rank's buffer is its 8 slices in order",
           "input_sha256_per_rank": shas,
           "output_sha256": outs[0],
           "output_note": "sha256 of any rank's buffer after the allreduce as the CPU oracle computes it (all ranks hold "
                          "the same bits); bit patterns of the bf16 values, little endian"}
    with open(os.path.join(ROOT, "tests", "golden", "headline_sha256.json"), "w") as f:
        json.dump(doc, f, indent=1)
        f.write("\n")
    return 0


if __name__ == "__main__":
    sys.exit(main())
