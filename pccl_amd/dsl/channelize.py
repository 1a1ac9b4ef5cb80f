"""Auto-channelisation of sequential chains and the cost model that decides it.

Reference: pccl/dsl/passes/channelize.py (the pass) and pccl/dsl/superopt/cost_model.py:47-200 (the
profile and the critical-path estimate).  The pass looks for chains of same-type data ops on
channel 0 whose source ranges follow one another, asks the cost model whether spreading the chain
over `num_channels` channels shortens the critical path, and if so relabels the ops' channels:
the first ceil(n / channels) ops stay on channel 0, the next block goes to channel 1, and so on.
Dependencies are not touched.

Profiles are plain data.  ``H100_PROFILE`` carries the reference's default figures so that the
pass takes the same decisions as the reference's on the same graph; ``MI355X_PROFILE`` carries what
this executor measures on one MI355X with virtual ranks: the payload rate of a local chunk copy
and of a chunk reduce, and the cost of one more dependency level (one more launch of the level
runner).  On one GPU all channels share the same HBM, so a channel is a label that orders
signals, not a separate path; the runner already executes independent ops of a level side by side
whatever their channels.
"""
from __future__ import annotations

from collections import defaultdict, deque
from dataclasses import dataclass, field
from typing import Dict, List, Optional, Sequence, Tuple

from .ir import Graph, Op

_SYNC = ("notify", "wait_notify", "noop")


@dataclass
class DeviceProfile:
    name: str = "h100"
    launch_overhead_us: float = 1.0
    bandwidth_gb_s: Dict[str, float] = field(default_factory=lambda: {
        "sm": 50.0, "tma": 60.0, "ce": 40.0, "rdma": 25.0, "multimem": 180.0, "host": 10.0})
    reduce_throughput_gops: Dict[str, float] = field(default_factory=lambda: {
        "sm": 30.0, "tma": 35.0, "multimem": 100.0})
    num_channels: int = 4
    per_channel_bw_gb_s: Dict[str, float] = field(default_factory=lambda: {
        "sm": 50.0, "tma": 60.0, "ce": 40.0, "rdma": 25.0, "multimem": 180.0, "host": 10.0})
    channel_launch_overhead_us: float = 0.5

    def to_dict(self) -> dict:
        return {"name": self.name, "launch_overhead_us": self.launch_overhead_us,
                "bandwidth_gb_s": self.bandwidth_gb_s, "reduce_throughput_gops": self.reduce_throughput_gops,
                "num_channels": self.num_channels, "per_channel_bw_gb_s": self.per_channel_bw_gb_s,
                "channel_launch_overhead_us": self.channel_launch_overhead_us}

    @classmethod
    def from_dict(cls, d: dict) -> "DeviceProfile":
        return cls(name=d.get("name", "custom"), launch_overhead_us=d.get("launch_overhead_us", 1.0),
                   bandwidth_gb_s=d.get("bandwidth_gb_s", {}),
                   reduce_throughput_gops=d.get("reduce_throughput_gops", {}),
                   num_channels=d.get("num_channels", 4), per_channel_bw_gb_s=d.get("per_channel_bw_gb_s", {}),
                   channel_launch_overhead_us=d.get("channel_launch_overhead_us", 0.5))


H100_PROFILE = DeviceProfile()

# One MI355X, virtual ranks in its HBM.  A chunk copy streams at 6.7 TB/s of traffic = 3.35 TB/s
# of payload; a chunk reduce (two reads, one write) at 6.6 TB/s of traffic = 2.2 TB/s of payload =
# 550 G four-byte elements per second; one more dependency level costs one more launch of the
# level runner (about 4.5 us back to back).  tma.* run as the sm.* ops.
MI355X_PROFILE = DeviceProfile(
    name="mi355x-vranks",
    launch_overhead_us=4.5,
    bandwidth_gb_s={"sm": 3350.0, "tma": 3350.0, "host": 10.0},
    reduce_throughput_gops={"sm": 550.0, "tma": 550.0},
    num_channels=8,
    per_channel_bw_gb_s={"sm": 3350.0, "tma": 3350.0, "host": 10.0},
    channel_launch_overhead_us=0.0,
)


def op_latency_us(primitive: str, profile: DeviceProfile, data_size_bytes: int = 0) -> float:
    """launch + transfer for a copy, launch + max(transfer, compute) for a reduce, launch for a
    signal (reference cost_model.py:113-140)."""
    launch = profile.launch_overhead_us
    if primitive in _SYNC:
        return launch
    executor = primitive.split(".", 1)[0]
    bw = profile.bandwidth_gb_s.get(executor, 10.0)
    transfer = data_size_bytes / (bw * 1e3) if bw > 0 else 0.0
    if primitive.endswith(".copy"):
        return launch + transfer
    if primitive.endswith(".reduce"):
        tp = profile.reduce_throughput_gops.get(executor, 30.0)
        compute = (data_size_bytes // 4) / (tp * 1e3) if tp > 0 else 0.0
        return launch + max(transfer, compute)
    return launch


def critical_path_cost_us(nodes: Sequence[Tuple[str, int]], edges: Sequence[Tuple[int, int]],
                          profile: DeviceProfile, data_size_bytes: int = 0) -> float:
    """Longest path through a pattern of (primitive, channel) nodes.  With more than one channel in
    use, consecutive nodes of one channel are serialised and every extra channel adds its launch
    overhead (reference cost_model.py:143-200)."""
    n = len(nodes)
    if n == 0:
        return 0.0
    channels = {c for _, c in nodes}
    lat = [op_latency_us(p, profile, data_size_bytes) for p, _ in nodes]
    adj: Dict[int, List[int]] = defaultdict(list)
    for a, b in edges:
        adj[a].append(b)
    if len(channels) > 1:
        for ch in channels:
            idx = [i for i in range(n) if nodes[i][1] == ch]
            for a, b in zip(idx, idx[1:]):
                if b not in adj[a]:
                    adj[a].append(b)
    indeg = [0] * n
    for u in range(n):
        for v in adj[u]:
            indeg[v] += 1
    finish = [0.0] * n
    ready = deque()
    for i in range(n):
        if indeg[i] == 0:
            finish[i] = lat[i]
            ready.append(i)
    while ready:
        u = ready.popleft()
        for v in adj[u]:
            finish[v] = max(finish[v], finish[u] + lat[v])
            indeg[v] -= 1
            if indeg[v] == 0:
                ready.append(v)
    cost = max(finish)
    if len(channels) > 1:
        cost += profile.channel_launch_overhead_us * (len(channels) - 1)
    return cost


class ChannelizePass:
    def __init__(self, num_channels: int = 2, min_data_size: int = 4096,
                 profile: DeviceProfile = H100_PROFILE):
        self.num_channels = num_channels
        self.min_data_size = min_data_size
        self.profile = profile

    def run(self, graph: Graph) -> Graph:
        graph.relink()
        for chain in self.find_chains(graph):
            self.try_channelize(chain)
        return graph

    # -- chains ---------------------------------------------------------------------------
    def find_chains(self, graph: Graph) -> List[List[Op]]:
        seen = set()
        chains = []
        for op in graph.topo_order():
            if op.uid in seen or not op.is_data or op.channel != 0:
                continue
            chain = [op]
            seen.add(op.uid)
            cur = op
            while True:
                nxt = self._next_data_op(graph, cur)
                if nxt is None or nxt.uid in seen or nxt.primitive != op.primitive or nxt.channel != 0:
                    break
                if not self._follows(cur, nxt):
                    break
                chain.append(nxt)
                seen.add(nxt.uid)
                cur = nxt
            if len(chain) > self.num_channels:
                chains.append(chain)
        return chains

    @staticmethod
    def _next_data_op(graph: Graph, op: Op) -> Optional[Op]:
        queue = deque(op.nexts)
        visited = set()
        while queue:
            u = queue.popleft()
            if u in visited:
                continue
            visited.add(u)
            nxt = graph.ops.get(u)
            if nxt is None:
                continue
            if nxt.primitive in _SYNC:
                queue.extend(nxt.nexts)
            elif nxt.is_data:
                return nxt
        return None

    @staticmethod
    def _extent(op: Op) -> int:
        return op.params.get("size", op.params.get("count", 0))

    def _follows(self, a: Op, b: Op) -> bool:
        key = "size" if "size" in a.params and "size" in b.params else \
              "count" if "count" in a.params and "count" in b.params else None
        if key is None:
            return False
        return b.params.get("src_offset", 0) == a.params.get("src_offset", 0) + a.params[key]

    # -- decision -------------------------------------------------------------------------
    def try_channelize(self, chain: List[Op]) -> bool:
        n, nc = len(chain), self.num_channels
        if n <= nc:
            return False
        total = sum(self._extent(o) for o in chain)
        if total < self.min_data_size:
            return False
        per_op = total // n
        single = critical_path_cost_us([(o.primitive, 0) for o in chain], [(i, i + 1) for i in range(n - 1)],
                                       self.profile, per_op)
        per_ch = (n + nc - 1) // nc
        nodes: List[Tuple[str, int]] = []
        edges: List[Tuple[int, int]] = []
        for ch in range(nc):
            lo, hi = ch * per_ch, min((ch + 1) * per_ch, n)
            first = len(nodes)
            nodes.extend((chain[j].primitive, ch) for j in range(lo, hi))
            edges.extend((first + j, first + j + 1) for j in range(hi - lo - 1))
        multi = critical_path_cost_us(nodes, edges, self.profile, per_op)
        if multi >= single:
            return False
        for i, o in enumerate(chain):
            o.channel = min(i // per_ch, nc - 1)
        return True
