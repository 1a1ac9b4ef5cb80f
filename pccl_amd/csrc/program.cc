// Cross-rank linker and plan builder.
//
// The reference runs one process per rank and lets counting semaphores order the ranks at run time
// (csrc/plugins/cuda/cuda_executor.cu:414-445).  With all ranks in one address space the same
// ordering can be derived once, on the host: simulate the semaphores, pair every wait with the
// notify that releases it, and keep only the resulting dependencies between data ops.
#include "program.h"

#include <algorithm>
#include <cstring>
#include <deque>
#include <map>
#include <numeric>
#include <set>

namespace pccl_hip {

namespace {

struct Bitset {
    std::vector<uint64_t> w;
    explicit Bitset(size_t n = 0) : w((n + 63) / 64, 0) {}
    void set(size_t i) { w[i >> 6] |= 1ull << (i & 63); }
    bool test(size_t i) const { return w[i >> 6] >> (i & 63) & 1; }
    void or_with(const Bitset& o) { for (size_t k = 0; k < w.size(); ++k) w[k] |= o.w[k]; }
};

struct Node {
    int rank, pos;
    std::vector<int> preds;  // global node ids
};

std::string op_name(const RankGraph& g, int rank, int pos) {
    const GraphOp& o = g.ops[pos];
    const char* k = o.kind == OpKind::Reduce ? "reduce" : o.kind == OpKind::Copy ? "copy" : o.kind == OpKind::Notify ? "notify" : o.kind == OpKind::Wait ? "wait_notify" : "noop";
    return "rank " + std::to_string(rank) + " op " + std::to_string(o.index) + " (" + k + ")";
}

constexpr size_t kClosureLimit = 24000;   // nodes; above this the O(N^2) checks are skipped
constexpr size_t kPairLimit = 20000000;   // access pairs examined by the race check

}  // namespace

// Last step of building a segment's column program: mark the last write of every rank and list
// the ranks the program reads by first touch (what a runner that keeps re-read values on chip
// has to fetch up front).
static void finish_column_program(Program& P, ColSegment& seg, std::vector<ColInstr>& prog) {
    uint64_t seen = 0;
    for (size_t n = prog.size(); n-- > 0;) {
        if (!(seen >> prog[n].self & 1)) prog[n].store |= STORE_LAST;
        seen |= 1ull << prog[n].self;
    }
    // Broadcast tail: allreduce-type programs end with a run of copies that all carry the same
    // value (the ring's allgather phase, the tree's broadcast).  Keep the first of them - after it
    // the accumulator holds that value - and turn the rest into one mask of ranks to store it to.
    {
        std::vector<int> cur(64);
        for (int r = 0; r < 64; ++r) cur[r] = r;          // value ids: the original contents
        int next_id = 64;
        std::vector<int> out(prog.size());
        for (size_t n = 0; n < prog.size(); ++n) {
            out[n] = prog[n].b_src == SRC_NONE ? cur[prog[n].peer] : next_id++;
            cur[prog[n].self] = out[n];
        }
        size_t s0 = prog.size();
        while (s0 > 0 && prog[s0 - 1].b_src == SRC_NONE && out[s0 - 1] == out[prog.size() - 1]) --s0;
        if (prog.size() - s0 >= 2) {
            uint64_t mask = 0;
            for (size_t n = s0 + 1; n < prog.size(); ++n) {
                const int kind = prog[n].store & STORE_KIND;
                if (kind == 2 || (kind == 1 && (prog[n].store & STORE_LAST))) mask |= 1ull << prog[n].self;
            }
            // the kept instruction: if a later copy of the run rewrites its rank (with the same
            // value) the mask covers that rank; otherwise a live store of it is a final one
            ColInstr& head = prog[s0];
            if (!(head.store & STORE_LAST)) head.store = 0;
            else if (head.store & STORE_KIND) head.store = (uint8_t)(2 | STORE_LAST);
            prog.resize(s0 + 1);
            seg.bcast_mask = mask;
        }
    }
    std::vector<uint8_t> pre;
    uint64_t listed = 0;
    auto want = [&](uint8_t r) { if (!(listed >> r & 1)) { listed |= 1ull << r; pre.push_back(r); } };
    for (const ColInstr& in : prog) {
        if (in.a_src == SRC_MEM && in.a_first) want(in.peer);
        if (in.b_src == SRC_MEM && in.b_first) want(in.self);
    }
    seg.pre_start = (int)P.col_pre.size();
    for (size_t i = 0; i < pre.size(); i += 8) {
        uint64_t w = ~0ull;
        for (size_t j = i; j < pre.size() && j < i + 8; ++j) w = (w & ~(0xFFull << (8 * (j - i)))) | ((uint64_t)pre[j] << (8 * (j - i)));
        P.col_pre.push_back(w);
    }
    seg.pre_words = (int)P.col_pre.size() - seg.pre_start;
    // pad with no-ops (acc = acc, nothing stored) so that a runner may read four instructions at
    // a time; programs start at multiples of four words because every program is padded
    ColInstr nop{};
    nop.a_src = SRC_ACC; nop.b_src = SRC_NONE;
    while (prog.size() % 4) prog.push_back(nop);
    seg.prog_len = (int)prog.size();
}

// Memory traffic of one segment under the two ways of running its program: every MEM operand
// loaded and every live store written (re-read values go through memory), or first touches
// fetched once and only final values written (re-read values stay on chip).
static void count_column_traffic(const Program& P, const ColSegment& seg, int es, int64_t* loads, int64_t* stores,
                                 int64_t* slot_loads, int64_t* slot_stores) {
    const int64_t bytes = (seg.end - seg.start) * es;
    for (int k = 0; k < seg.prog_len; ++k) {
        const ColInstr& in = P.col_instrs[seg.prog_start + k];
        const int kind = in.store & STORE_KIND;
        if (in.a_src == SRC_MEM) *loads += bytes;
        if (in.b_src == SRC_MEM) *loads += bytes;
        if (kind) *stores += bytes;
        if (kind == 2 || (kind == 1 && (in.store & STORE_LAST))) *slot_stores += bytes;
    }
    const int tail = __builtin_popcountll(seg.bcast_mask);
    *stores += bytes * tail;
    *slot_stores += bytes * tail;
    for (int w = 0; w < seg.pre_words; ++w)
        for (int j = 0; j < 8; ++j)
            if ((P.col_pre[seg.pre_start + w] >> (8 * j) & 0xFF) != 0xFF) *slot_loads += bytes;
}

// The chain form of a finished column program, if it has one (see ChainSegment).  The program is
// evaluated symbolically: every value is a leaf (the original content of a rank) or the combination
// of two values.  It is a chain when all ranks that are written to memory end up holding one and the
// same value and that value combines every leaf at most once, either literally as a chain (each
// combination takes one leaf and the chain so far: any element type and operator, the order is kept)
// or in any shape under an operator whose result does not depend on the order for this element
// type: wrapping integer addition, and maximum / minimum of any type (IEEE 754-2019 maximum and
// minimum are associative and commutative, signed zeros and NaN - written canonically - included),
// or - third form, reported through depth_out - as a perfectly balanced binary tree, whose shape is
// kept (floating-point sums of halving-doubling and tree schedules).
// Operand order within one combination never matters: every operator here is commutative bit for bit.
static bool chain_form(const Program& P, const ColSegment& seg, int dtype, std::vector<uint8_t>* srcs, int* redop_out, uint64_t* mask_out, int* depth_out) {
    *depth_out = 0;
    struct Val { int a = -1, b = -1, leaf = -1, redop = 0; };   // leaf >= 0: original content of that rank
    std::vector<Val> vals;
    std::vector<int> cur(PCCL_HIP_MAX_VRANKS);
    for (int r = 0; r < PCCL_HIP_MAX_VRANKS; ++r) { Val v; v.leaf = r; vals.push_back(v); cur[r] = r; }
    std::vector<int> final_of(PCCL_HIP_MAX_VRANKS, -1);
    int acc = -1;
    for (int k = 0; k < seg.prog_len; ++k) {
        const ColInstr& in = P.col_instrs[seg.prog_start + k];
        const int a = in.a_src == SRC_ACC ? acc : cur[in.peer];
        int res = a;
        if (in.b_src != SRC_NONE) {
            const int b = in.b_src == SRC_ACC ? acc : cur[in.self];
            if (a < 0 || b < 0) return false;
            Val v; v.a = a; v.b = b; v.redop = in.redop;
            vals.push_back(v);
            res = (int)vals.size() - 1;
        }
        if (res < 0) continue;   // padding in front of any value (never produced by the planner)
        acc = res;
        const int kind = in.store & STORE_KIND;
        if (kind) cur[in.self] = res;
        if (kind == 2 || (kind == 1 && (in.store & STORE_LAST))) final_of[in.self] = res;
    }
    for (uint64_t m = seg.bcast_mask; m; m &= m - 1) final_of[__builtin_ctzll(m)] = acc;
    int root = -1;
    uint64_t mask = 0;
    for (int r = 0; r < PCCL_HIP_MAX_VRANKS; ++r) {
        if (final_of[r] < 0) continue;
        if (root >= 0 && final_of[r] != root) return false;     // different values in different ranks
        root = final_of[r];
        mask |= 1ull << r;
    }
    if (root < 0) return false;
    // flatten the root: leaves in chain order, one operator throughout
    int redop = -1;
    bool literal = true;          // every combination takes at least one leaf
    std::vector<uint8_t> leaves;
    std::vector<int> stack = {root};
    // literal chains are walked from the root down: the leaf of each combination is met before the
    // rest of the chain, so the list comes out last-combined first and is reversed at the end
    while (!stack.empty()) {
        const int id = stack.back(); stack.pop_back();
        const Val& v = vals[id];
        if (v.leaf >= 0) { leaves.push_back((uint8_t)v.leaf); continue; }
        if (redop >= 0 && v.redop != redop) return false;
        redop = v.redop;
        const bool la = vals[v.a].leaf >= 0, lb = vals[v.b].leaf >= 0;
        if (!la && !lb) literal = false;
        // push the deeper side first so that it is popped last: [leaf now, rest later]
        if (la) { stack.push_back(v.b); stack.push_back(v.a); }
        else { stack.push_back(v.a); stack.push_back(v.b); }
    }
    std::reverse(leaves.begin(), leaves.end());
    uint64_t seen = 0;
    for (uint8_t r : leaves) { if (seen >> r & 1) return false; seen |= 1ull << r; }
    if (!literal) {
        const bool free_order = redop == PCCL_MAX || redop == PCCL_MIN || (redop == PCCL_SUM && dtype == PCCL_I32);
        if (free_order) std::sort(leaves.begin(), leaves.end());
        else {
            // the shape matters: accept a perfectly balanced tree, leaves listed left to right
            struct Walk {
                const std::vector<Val>& vals;
                std::vector<uint8_t> out;
                int depth_of(int id) {          // depth of a perfect subtree, -1 if it is not perfect
                    const Val& v = vals[id];
                    if (v.leaf >= 0) { out.push_back((uint8_t)v.leaf); return 0; }
                    const int da = depth_of(v.a);
                    if (da < 0) return -1;
                    const int db = depth_of(v.b);
                    return db == da ? da + 1 : -1;
                }
            } walk{vals, {}};
            const int depth = walk.depth_of(root);
            if (depth < 1 || depth > 6) return false;
            leaves = walk.out;
            *depth_out = depth;
        }
    }
    *srcs = leaves; *redop_out = redop < 0 ? PCCL_SUM : redop; *mask_out = mask;
    return true;
}

// Chain forms of all segments of a plan, or none.
static void plan_chains(Program& P, const std::vector<ColSegment>& segs, std::vector<ChainSegment>* out) {
    out->clear();
    std::vector<ChainSegment> chains;
    const size_t srcs_before = P.chain_srcs.size();
    for (const ColSegment& seg : segs) {
        std::vector<uint8_t> srcs;
        int redop = PCCL_SUM, depth = 0;
        uint64_t mask = 0;
        if (!chain_form(P, seg, P.dtype, &srcs, &redop, &mask, &depth)) { P.chain_srcs.resize(srcs_before); return; }
        ChainSegment c;
        c.start = seg.start; c.end = seg.end; c.redop = redop; c.store_mask = mask; c.tree_depth = depth;
        c.src_start = (int32_t)P.chain_srcs.size(); c.n_src = (int32_t)srcs.size();
        P.chain_srcs.insert(P.chain_srcs.end(), srcs.begin(), srcs.end());
        chains.push_back(c);
    }
    *out = std::move(chains);
}

std::vector<SignalUse> signal_uses(const std::vector<const RankGraph*>& graphs) {
    std::map<std::pair<int, int>, SignalUse> uses;
    for (size_t r = 0; r < graphs.size(); ++r) {
        if (!graphs[r]) continue;
        for (const GraphOp& o : graphs[r]->ops) {
            if (o.kind != OpKind::Wait && o.kind != OpKind::Notify) continue;
            const auto key = std::make_pair(o.kind == OpKind::Wait ? (int)r : (int)o.peer, (int)o.off0);
            SignalUse& u = uses[key];
            u.rank = key.first; u.id = key.second;
            (o.kind == OpKind::Wait ? u.waits : u.notifies) += 1;
        }
    }
    std::vector<SignalUse> out;
    for (const auto& kv : uses) out.push_back(kv.second);
    return out;
}

// The linker: R per-rank graphs in, one Program out.  Each step is a method; they run in the order
// `run` calls them and hand their results on through the members.
namespace {

class Linker {
  public:
    Linker(const std::vector<const RankGraph*>& graphs_, const LinkOptions& opt_)
        : graphs(graphs_), opt(opt_), R((int)graphs_.size()) {}

    Program run() {
        read_headers();
        check_ranks();
        simulate_semaphores();
        build_reachability();
        collect_data_ops();
        check_races();
        keep_conflict_dependencies();
        order_ops();
        plan_steps();
        plan_gather();
        plan_column();
        plan_direct();
        return std::move(P);
    }

  private:
    const std::vector<const RankGraph*>& graphs;
    const LinkOptions& opt;
    const int R;
    Program P;
    std::vector<int> base;          // node id of rank r's op i = base[r] + i
    int N = 0;                      // ops of all ranks, signals included
    int es = 0;                     // element size in bytes
    std::vector<Node> nodes;        // happens-before graph over all ops
    std::vector<int> exec_order;    // one execution order the semaphores allow (a topological order)
    std::map<std::pair<int, int>, std::vector<int>> notify_seq, wait_seq;   // per (rank, signal id), for the ambiguity check
    bool closure = false;           // reach[] is available (the graph is small enough for N^2 bits)
    std::vector<Bitset> reach;      // reach[v] = nodes that happen before v
    std::vector<int> data_of;       // node id -> provisional data-op index (-1: a signal or noop)
    std::vector<int> data_nodes;    // provisional data-op index -> node id
    int D = 0;                      // number of data ops
    std::vector<LinkedOp> ops;      // data ops in execution order, before the final sort
    std::vector<std::vector<ColInstr>> raw_progs;   // column plan: per segment, before finish_column_program


    void read_headers() {
        if (R <= 0 || R > PCCL_HIP_MAX_VRANKS) throw Error{PCCL_ERR_INVALID, "number of virtual ranks must be 1.." + std::to_string(PCCL_HIP_MAX_VRANKS)};
        P.R = R;
        bool have_dtype = false;
        base.assign(R + 1, 0);
        for (int r = 0; r < R; ++r) {
            if (!graphs[r]) throw Error{PCCL_ERR_LINK, "virtual rank " + std::to_string(r) + " has no registered graph"};
            const RankGraph& g = *graphs[r];
            base[r + 1] = base[r] + (int)g.ops.size();
            if (g.has_dtype) {
                if (have_dtype && g.dtype != P.dtype) throw Error{PCCL_ERR_LINK, "ranks disagree on tensor_info.dtype"};
                P.dtype = g.dtype; have_dtype = true;
            }
            if (r == 0) { P.collective_type = g.collective_type; P.tensor_elems = g.tensor_elems; }
            else if (g.collective_type != P.collective_type) throw Error{PCCL_ERR_LINK, "ranks disagree on collective_type"};
            P.buffer_elems = std::max(P.buffer_elems, g.max_extent());
            P.tensor_elems = std::max(P.tensor_elems, g.tensor_elems);
        }
        N = base[R];
        P.num_all_ops = N;
        es = elem_size(P.dtype);
    }

    void check_ranks() {
        for (int r = 0; r < R; ++r)
            for (size_t i = 0; i < graphs[r]->ops.size(); ++i) {
                const GraphOp& o = graphs[r]->ops[i];
                bool uses_peer = o.kind == OpKind::Reduce || o.kind == OpKind::Copy || o.kind == OpKind::Notify;
                if (uses_peer && (o.peer < 0 || o.peer >= R))
                    throw Error{PCCL_ERR_LINK, op_name(*graphs[r], r, (int)i) + " names rank " + std::to_string(o.peer) + " but only " + std::to_string(R) + " virtual ranks exist"};
            }
    }

    // Simulate the semaphores with the discipline of the reference's dependency-counter runner: per
    // rank and channel a FIFO of ready ops, one at a time; a wait blocks its channel.
    void simulate_semaphores() {
        nodes.assign(N, Node{});
        for (int r = 0; r < R; ++r)
            for (size_t i = 0; i < graphs[r]->ops.size(); ++i) {
                Node& n = nodes[base[r] + i];
                n.rank = r; n.pos = (int)i;
                for (int d : graphs[r]->ops[i].deps) n.preds.push_back(base[r] + d);
            }
        std::vector<int> remaining(N);
        std::vector<std::deque<int>> queues((size_t)R * PCCL_HIP_MAX_CHANNELS);
        for (int r = 0; r < R; ++r)
            for (size_t i = 0; i < graphs[r]->ops.size(); ++i) {
                remaining[base[r] + i] = graphs[r]->ops[i].num_deps_declared;
                if (remaining[base[r] + i] == 0) queues[(size_t)r * PCCL_HIP_MAX_CHANNELS + graphs[r]->ops[i].channel].push_back((int)i);
            }
        // per (target rank, id): notify nodes not yet consumed, in arrival order
        std::map<std::pair<int, int>, std::deque<int>> pending;
        // counts carried in from earlier executions: a wait takes one of these before it takes a notify
        // of this execution (the waits on one semaphore are ordered among themselves, so the first
        // ones are the ones that pass unconditionally at run time too)
        std::map<std::pair<int, int>, int> credit;
        for (const auto& c : opt.carried)
            if (c.second > 0) credit[c.first] += c.second;
        exec_order.reserve(N);
        int done = 0;
        while (done < N) {
            bool progressed = false;
            for (int r = 0; r < R; ++r)
                for (int c = 0; c < PCCL_HIP_MAX_CHANNELS; ++c) {
                    auto& q = queues[(size_t)r * PCCL_HIP_MAX_CHANNELS + c];
                    while (!q.empty()) {
                        int i = q.front();
                        const GraphOp& o = graphs[r]->ops[i];
                        int id = base[r] + i;
                        if (o.kind == OpKind::Wait) {
                            auto key = std::make_pair(r, (int)o.off0);
                            auto cr = credit.find(key);
                            if (cr != credit.end() && cr->second > 0) {
                                --cr->second;                    // passes on a carried count: ordered after nothing here
                                ++P.carried_waits;
                            } else {
                                auto it = pending.find(key);
                                if (it == pending.end() || it->second.empty()) break;  // blocked
                                nodes[id].preds.push_back(it->second.front());
                                it->second.pop_front();
                            }
                            wait_seq[key].push_back(id);
                        } else if (o.kind == OpKind::Notify) {
                            auto key = std::make_pair(o.peer, (int)o.off0);
                            pending[key].push_back(id);
                            notify_seq[key].push_back(id);
                        }
                        q.pop_front();
                        exec_order.push_back(id);
                        ++done; progressed = true;
                        for (int nx : o.nexts)
                            if (--remaining[base[r] + nx] == 0)
                                queues[(size_t)r * PCCL_HIP_MAX_CHANNELS + graphs[r]->ops[nx].channel].push_back(nx);
                    }
                }
            if (!progressed) {
                std::string blocked;
                int shown = 0;
                for (int r = 0; r < R && shown < 4; ++r)
                    for (int c = 0; c < PCCL_HIP_MAX_CHANNELS && shown < 4; ++c) {
                        auto& q = queues[(size_t)r * PCCL_HIP_MAX_CHANNELS + c];
                        if (!q.empty()) { blocked += (shown ? "; " : "") + op_name(*graphs[r], r, q.front()) + " waits on signal " + std::to_string(graphs[r]->ops[q.front()].off0); ++shown; }
                    }
                if (blocked.empty()) blocked = "ops with unmet dependencies (cyclic or dangling dependency lists)";
                throw Error{PCCL_ERR_LINK, "deadlock: " + std::to_string(done) + " of " + std::to_string(N) + " ops can run; blocked: " + blocked};
            }
        }
        std::vector<const RankGraph*> gs(graphs.begin(), graphs.end());
        P.signals = signal_uses(gs);
        for (const SignalUse& u : P.signals) if (u.notifies != u.waits) P.residual_signals++;
    }

    // Reachability (happens-before) over all ops, in execution order.
    void build_reachability() {
        closure = (size_t)N <= kClosureLimit;
        P.order_checked = closure;
        if (closure) {
            reach.assign(N, Bitset(N));
            for (int id : exec_order)
                for (int p : nodes[id].preds) { reach[id].or_with(reach[p]); reach[id].set(p); }
            auto ordered_seq = [&](const std::vector<int>& seq) {
                for (size_t k = 1; k < seq.size(); ++k)
                    if (!reach[seq[k]].test(seq[k - 1])) return false;
                return true;
            };
            for (auto& kv : notify_seq)
                if (!ordered_seq(kv.second))
                    throw Error{PCCL_ERR_LINK, "signal " + std::to_string(kv.first.second) + " of rank " + std::to_string(kv.first.first) + " is notified by ops that are not ordered with each other: the pairing of notifies and waits is ambiguous"};
            for (auto& kv : wait_seq)
                if (!ordered_seq(kv.second))
                    throw Error{PCCL_ERR_LINK, "signal " + std::to_string(kv.first.second) + " of rank " + std::to_string(kv.first.first) + " is awaited by ops that are not ordered with each other: the pairing of notifies and waits is ambiguous"};
        }
    }

    // The data ops and their nearest data predecessors (signals and noops contracted).
    void collect_data_ops() {
        data_of.assign(N, -1);
        for (int id : exec_order) {
            const GraphOp& o = graphs[nodes[id].rank]->ops[nodes[id].pos];
            if (o.kind == OpKind::Reduce || o.kind == OpKind::Copy) { data_of[id] = (int)data_nodes.size(); data_nodes.push_back(id); }
        }
        D = (int)data_nodes.size();
        // frontier[v] = set of data nodes that are the nearest data ancestors of v (through signals/noops)
        std::vector<std::vector<int>> frontier(N);
        for (int id : exec_order) {
            std::vector<int>& f = frontier[id];
            for (int p : nodes[id].preds) {
                if (data_of[p] >= 0) f.push_back(p);
                else f.insert(f.end(), frontier[p].begin(), frontier[p].end());
            }
            std::sort(f.begin(), f.end());
            f.erase(std::unique(f.begin(), f.end()), f.end());
            if (closure && f.size() > 1) {  // drop ancestors of other members
                std::vector<int> keep;
                for (int a : f) {
                    bool redundant = false;
                    for (int b : f) if (a != b && reach[b].test(a)) { redundant = true; break; }
                    if (!redundant) keep.push_back(a);
                }
                f.swap(keep);
            }
        }
        ops.assign(D, LinkedOp{});
        for (int k = 0; k < D; ++k) {
            int id = data_nodes[k];
            const GraphOp& o = graphs[nodes[id].rank]->ops[nodes[id].pos];
            LinkedOp& L = ops[k];
            L.rank = nodes[id].rank; L.channel = o.channel; L.graph_pos = nodes[id].pos; L.index = o.index;
            L.is_reduce = o.kind == OpKind::Reduce; L.redop = o.redop; L.peer = o.peer;
            L.off0 = o.off0; L.off1 = o.off1; L.off2 = o.off2; L.size = o.size;
            for (int p : frontier[id]) L.deps.push_back(data_of[p]);
            int lvl = 0;
            for (int d : L.deps) lvl = std::max(lvl, ops[d].level + 1);
            L.level = lvl;
            P.num_levels = std::max(P.num_levels, lvl + 1);
            P.algorithmic_bytes += (L.is_reduce ? 3 : 2) * L.size * es;
            // an op whose own source and destination ranges overlap without coinciding has no
            // defined element order
            auto partial = [&](int64_t s, int64_t d) { return s != d && s < d + L.size && d < s + L.size; };
            if (L.size > 0) {
                if (L.is_reduce && partial(L.off1, L.off2)) throw Error{PCCL_ERR_LINK, op_name(*graphs[L.rank], L.rank, L.graph_pos) + ": src and dst ranges overlap without coinciding"};
                if (L.peer == L.rank && partial(L.off0, L.dst_off())) throw Error{PCCL_ERR_LINK, op_name(*graphs[L.rank], L.rank, L.graph_pos) + ": reads and writes overlapping ranges of its own buffer"};
            }
        }
    }

    // Conflicting accesses to one rank buffer must be ordered by some notify / wait chain.
    void check_races() {
        if (opt.check_races && closure && D <= 1) P.race_checked = true;   // nothing to conflict with
        if (opt.check_races && closure && D > 1) {
            struct Acc { int rank; int64_t s, e; bool write; int op; };
            std::vector<Acc> acc;
            for (int k = 0; k < D; ++k) {
                const LinkedOp& L = ops[k];
                if (L.size <= 0) continue;
                acc.push_back({L.peer, L.off0, L.off0 + L.size, false, k});
                if (L.is_reduce) acc.push_back({L.rank, L.off1, L.off1 + L.size, false, k});
                acc.push_back({L.rank, L.dst_off(), L.dst_off() + L.size, true, k});
            }
            std::sort(acc.begin(), acc.end(), [](const Acc& a, const Acc& b) { return a.rank != b.rank ? a.rank < b.rank : a.s < b.s; });
            size_t pairs = 0;
            bool complete = true;
            for (size_t i = 0; i < acc.size() && complete; ++i)
                for (size_t j = i + 1; j < acc.size() && acc[j].rank == acc[i].rank && acc[j].s < acc[i].e; ++j) {
                    if (++pairs > kPairLimit) { complete = false; break; }
                    if (!(acc[i].write || acc[j].write) || acc[i].op == acc[j].op) continue;
                    int a = data_nodes[acc[i].op], b = data_nodes[acc[j].op];
                    if (!reach[a].test(b) && !reach[b].test(a)) {
                        const LinkedOp &A = ops[acc[i].op], &B = ops[acc[j].op];
                        throw Error{PCCL_ERR_LINK, "data race on rank " + std::to_string(acc[i].rank) + " elements [" + std::to_string(std::max(acc[i].s, acc[j].s)) + ", " + std::to_string(std::min(acc[i].e, acc[j].e)) + "): " +
                                                       op_name(*graphs[A.rank], A.rank, A.graph_pos) + " and " + op_name(*graphs[B.rank], B.rank, B.graph_pos) + " are not ordered by any notify/wait chain"};
                    }
                }
            P.race_checked = complete;
        }
    }

    // ---- keep only the orderings that matter: B must follow A exactly when A happens before B
    //      AND they touch overlapping memory with at least one write.  Chain order between ops on
    //      disjoint ranges (e.g. the ragged pieces of one schedule step) is not a dependency, so
    //      such ops share a level and run in one launch.  Any execution that respects these edges
    //      gives the results of every order the notify/wait chains allow.
    void keep_conflict_dependencies() {
        if (opt.conflict_deps && closure && D > 1 && D <= 8192) {
            auto overlaps = [](int64_t s0, int64_t n0, int64_t s1, int64_t n1) { return s0 < s1 + n1 && s1 < s0 + n0; };
            auto conflict = [&](const LinkedOp& A, const LinkedOp& B) {
                if (A.size <= 0 || B.size <= 0) return false;
                // writes of A against every access of B, and writes of B against reads of A
                if (A.rank == B.rank && overlaps(A.dst_off(), A.size, B.dst_off(), B.size)) return true;
                if (A.rank == B.peer && overlaps(A.dst_off(), A.size, B.off0, B.size)) return true;
                if (B.is_reduce && A.rank == B.rank && overlaps(A.dst_off(), A.size, B.off1, B.size)) return true;
                if (B.rank == A.peer && overlaps(B.dst_off(), B.size, A.off0, A.size)) return true;
                if (A.is_reduce && A.rank == B.rank && overlaps(B.dst_off(), B.size, A.off1, A.size)) return true;
                return false;
            };
            std::vector<Bitset> kept(D, Bitset(D));   // data ops ordered before k through kept edges
            P.num_levels = 0;
            for (int k = 0; k < D; ++k) {             // ops[] is in execution (topological) order
                LinkedOp& B = ops[k];
                B.deps.clear();
                for (int a = k - 1; a >= 0; --a) {    // latest first, so covered ancestors are skipped
                    if (kept[k].test(a)) continue;
                    if (!reach[data_nodes[k]].test(data_nodes[a]) || !conflict(ops[a], B)) continue;
                    B.deps.push_back(a);
                    kept[k].or_with(kept[a]);
                    kept[k].set(a);
                }
                int lvl = 0;
                for (int d : B.deps) lvl = std::max(lvl, ops[d].level + 1);
                B.level = lvl;
                P.num_levels = std::max(P.num_levels, lvl + 1);
            }
        }
    }

    // Final order: (level, rank, channel, graph position); dependencies renumbered to it.
    void order_ops() {
        std::vector<int> perm(D);
        std::iota(perm.begin(), perm.end(), 0);
        std::stable_sort(perm.begin(), perm.end(), [&](int a, int b) {
            const LinkedOp &A = ops[a], &B = ops[b];
            if (A.level != B.level) return A.level < B.level;
            if (A.rank != B.rank) return A.rank < B.rank;
            if (A.channel != B.channel) return A.channel < B.channel;
            return A.graph_pos < B.graph_pos;
        });
        std::vector<int> inv(D);
        for (int k = 0; k < D; ++k) inv[perm[k]] = k;
        P.ops.resize(D);
        for (int k = 0; k < D; ++k) {
            P.ops[k] = ops[perm[k]];
            for (int& d : P.ops[k].deps) d = inv[d];
            std::sort(P.ops[k].deps.begin(), P.ops[k].deps.end());
        }
    }

    // The stepwise plan: every op cut into work items.
    void plan_steps() {
        int64_t tile_bytes = opt.step_tile_bytes;
        if (tile_bytes <= 0) {
            // automatic: 32 KiB items (the fastest on large programs), halved down to 4 KiB while an
            // average level has fewer than 1024 items - a small program is bound by the latency of its
            // chain of levels, and needs its few bytes spread over many workgroups
            int64_t bytes = 0;
            for (const LinkedOp& L : P.ops) bytes += L.size * es;
            const int64_t per_level = bytes / std::max(1, P.num_levels);
            tile_bytes = 32 * 1024;
            while (tile_bytes > 4096 && per_level / tile_bytes < 1024) tile_bytes >>= 1;
        }
        P.tile_elems = std::max<int64_t>(tile_bytes / es, 1024);
        P.step_ops.resize(D);
        int64_t items = 0;
        for (int k = 0; k < D; ++k) {
            StepOpPlan& s = P.step_ops[k];
            s.first_item = (int)items;
            // the item grid is anchored at a multiple of the tile size in the destination buffer, so
            // that an op with an odd start still has whole, aligned items everywhere but at its ends
            const int64_t dst = P.ops[k].is_reduce ? P.ops[k].off2 : P.ops[k].off1;
            s.lead = (int)(dst % P.tile_elems);
            s.ntiles = (int)((P.ops[k].size + s.lead + P.tile_elems - 1) / P.tile_elems);
            s.dep_start = (int)P.step_deps.size();
            s.ndeps = (int)P.ops[k].deps.size();
            for (int d : P.ops[k].deps) P.step_deps.push_back(d);
            items += s.ntiles;
            if (items > INT32_MAX) throw Error{PCCL_ERR_UNSUPPORTED, "program has more than 2^31 work items"};
        }
        P.num_items = items;
    }

    // ---- gather plan: an alltoall graph whose ops are all copies out of regions nobody writes.
    // Staged semantics (reference engine_c.cc:524-543): input r sits at [0, n) of buffer r, the
    // program runs, output r is chunk r of the input region followed, for every other rank p, by
    // the scratch chunk [n + p*chunk, n + (p+1)*chunk).  Composing that with the copies gives, for
    // every output element, the input element it comes from - no buffer needed.  Abandoned (the
    // call then stages through the rank buffers) if any output element would come from scratch the
    // program never wrote, or if an op writes something another op reads or writes.
    void plan_gather() {
        if (P.collective_type == "alltoall" && D > 0 && P.tensor_elems > 0 && P.tensor_elems % R == 0) {
            const int64_t n = P.tensor_elems, chunk = n / R;
            bool ok = true;
            for (const LinkedOp& L : P.ops) if (L.is_reduce) ok = false;
            // sources inside the input region, destinations outside it and mutually disjoint per rank
            std::vector<std::vector<std::pair<int64_t, int>>> writes(R);   // (dst offset, op) per rank
            for (int k = 0; k < D && ok; ++k) {
                const LinkedOp& L = P.ops[k];
                if (L.size <= 0) continue;
                if (L.off0 < 0 || L.off0 + L.size > n || L.off1 < n) ok = false;
                writes[L.rank].push_back({L.off1, k});
            }
            for (int r = 0; r < R && ok; ++r) {
                std::sort(writes[r].begin(), writes[r].end());
                for (size_t i = 1; i < writes[r].size(); ++i) {
                    const LinkedOp& prev = P.ops[writes[r][i - 1].second];
                    if (prev.off1 + prev.size > writes[r][i].first) ok = false;
                }
            }
            for (int r = 0; r < R && ok; ++r)
                for (int p = 0; p < R && ok; ++p) {
                    if (p == r) { P.gather.push_back({r, r, (int64_t)p * chunk, (int64_t)r * chunk, chunk}); continue; }
                    int64_t x = n + (int64_t)p * chunk;
                    const int64_t x_end = x + chunk;
                    while (x < x_end && ok) {        // walk the scratch chunk through the ops that wrote it
                        const LinkedOp* hit = nullptr;
                        for (auto& w : writes[r]) {
                            const LinkedOp& L = P.ops[w.second];
                            if (L.off1 <= x && x < L.off1 + L.size) { hit = &L; break; }
                        }
                        if (!hit) { ok = false; break; }
                        const int64_t len = std::min(x_end, hit->off1 + hit->size) - x;
                        P.gather.push_back({r, hit->peer, (int64_t)p * chunk + (x - (n + (int64_t)p * chunk)), hit->off0 + (x - hit->off1), len});
                        x += len;
                    }
                }
            if (!ok) P.gather.clear();
        }
    }

    // The column program of one segment: the ops covering it in program order, values forwarded
    // through the accumulator where one op's result is the next one's operand, dead stores dropped,
    // final stores marked (not yet finished: see finish_column_program).
    std::vector<ColInstr> segment_program(const std::vector<int>& covering) const {
        std::vector<ColInstr> prog;
        uint64_t written = 0;  // ranks an earlier instruction of this program wrote
        for (size_t n = 0; n < covering.size(); ++n) {
            const LinkedOp& L = P.ops[covering[n]];
            ColInstr in{};
            in.self = (uint8_t)L.rank; in.peer = (uint8_t)L.peer; in.redop = (uint8_t)L.redop; in.store = 1;
            bool prev_is_peer = n > 0 && prog.back().self == in.peer;
            bool prev_is_self = n > 0 && prog.back().self == in.self;
            in.a_src = prev_is_peer ? SRC_ACC : SRC_MEM;
            in.b_src = !L.is_reduce ? SRC_NONE : prev_is_self ? SRC_ACC : SRC_MEM;
            if (in.a_src == SRC_MEM) in.a_first = !(written >> in.peer & 1);
            if (in.b_src == SRC_MEM) in.b_first = !(written >> in.self & 1);
            written |= 1ull << in.self;
            prog.push_back(in);
        }
        // dead stores: overwritten before any later instruction reads that rank from memory
        for (size_t n = 0; n < prog.size(); ++n) {
            for (size_t m = n + 1; m < prog.size(); ++m) {
                bool reads = (prog[m].a_src != SRC_ACC && prog[m].peer == prog[n].self) ||
                             (prog[m].b_src == SRC_MEM && prog[m].self == prog[n].self);
                if (reads) break;
                if (prog[m].self == prog[n].self) { prog[n].store = 0; break; }
            }
        }
        // a store nothing in this program reads back from memory is final: mark it streaming
        for (size_t n = 0; n < prog.size(); ++n) {
            if (!prog[n].store) continue;
            bool reread = false;
            for (size_t m = n + 1; m < prog.size() && !reread; ++m)
                reread = (prog[m].a_src != SRC_ACC && prog[m].peer == prog[n].self) ||
                         (prog[m].b_src == SRC_MEM && prog[m].self == prog[n].self);
            if (!reread) prog[n].store = 2;
        }
        return prog;
    }

    // The column plan: when every op reads and writes the same element positions, the program
    // decomposes by position into segments with one column program each.
    void plan_column() {
        P.position_aligned = D > 0;
        for (auto& L : P.ops) if (!L.position_aligned()) { P.position_aligned = false; break; }
        if (P.position_aligned) {
            std::vector<int64_t> cuts;
            for (auto& L : P.ops) if (L.size > 0) { cuts.push_back(L.off0); cuts.push_back(L.off0 + L.size); }
            std::sort(cuts.begin(), cuts.end());
            cuts.erase(std::unique(cuts.begin(), cuts.end()), cuts.end());
            // ops covering each elementary interval, in program order
            std::vector<std::vector<int>> cover(cuts.size() > 0 ? cuts.size() - 1 : 0);
            for (int k = 0; k < D; ++k) {
                const LinkedOp& L = P.ops[k];
                if (L.size <= 0) continue;
                size_t a = std::lower_bound(cuts.begin(), cuts.end(), L.off0) - cuts.begin();
                size_t b = std::lower_bound(cuts.begin(), cuts.end(), L.off0 + L.size) - cuts.begin();
                for (size_t i = a; i < b; ++i) cover[i].push_back(k);
            }
            // instruction signature of an op list (what the device program depends on)
            auto sig = [&](const std::vector<int>& v) {
                std::vector<int> s;
                for (int k : v) { const LinkedOp& L = P.ops[k]; s.push_back(L.rank | L.peer << 8 | (int)L.is_reduce << 16 | L.redop << 17); }
                return s;
            };
            std::vector<int> prev_sig;
            for (size_t i = 0; i < cover.size(); ++i) {
                if (cover[i].empty()) { prev_sig.clear(); continue; }
                std::vector<int> s = sig(cover[i]);
                if (!P.segs.empty() && P.segs.back().end == cuts[i] && s == prev_sig) { P.segs.back().end = cuts[i + 1]; continue; }
                prev_sig = s;
                ColSegment seg;
                seg.start = cuts[i]; seg.end = cuts[i + 1];
                seg.prog_start = (int)P.col_instrs.size();
                std::vector<ColInstr> prog = segment_program(cover[i]);
                seg.prog_len = (int)prog.size();
                raw_progs.push_back(prog);            // the direct plan below starts from the unfinished form
                finish_column_program(P, seg, prog);
                P.col_instrs.insert(P.col_instrs.end(), prog.begin(), prog.end());
                P.segs.push_back(seg);
            }
            for (auto& seg : P.segs)
                count_column_traffic(P, seg, es, &P.column_load_bytes, &P.column_store_bytes, &P.slot_load_bytes, &P.slot_store_bytes);
            plan_chains(P, P.segs, &P.chain_segs);
        }
    }

    // ---- direct plan: the same programs with the caller's input tensors as the source of
    // every first-touch load and the output tensors as the destination of every store, so
    // that no staging copy is needed.  The staged semantics are "place input r in buffer r at
    // its window, run, hand back the output window of buffer r" (reference engine_c.cc:468-548):
    //   allreduce / untyped   in [0,n)                out [0,n)
    //   reduce_scatter        in [0,n)                out [r*n/R, (r+1)*n/R)
    //   allgather             in [r*n/R, (r+1)*n/R)   out [0,n)
    // For the result to be identical, a (rank, position) inside the output window that the
    // program never writes is passed through from the input (one copy instruction with
    // peer = self), a final store outside the output window is dropped (nobody can observe
    // it), and the plan is abandoned (staging is used instead) if any access would need
    // memory outside the windows: a first touch outside the input window, or a value that is
    // written outside the output window and read back later.
    void plan_direct() {
        if (!P.position_aligned) return;
        const int64_t n = P.tensor_elems;
        const std::string& ct = P.collective_type;
        const bool ar = ct.empty() || ct == "allreduce";
        const bool rs = ct == "reduce_scatter", ag = ct == "allgather";
        if ((ar || rs || ag) && n >= P.buffer_elems && n > 0 && (ar || n % R == 0)) {
            const int64_t chunk = n / R;
            P.direct_in_start.assign(R, 0); P.direct_in_end.assign(R, n);
            P.direct_out_start.assign(R, 0); P.direct_out_end.assign(R, n);
            for (int r = 0; r < R; ++r) {
                if (rs) { P.direct_out_start[r] = r * chunk; P.direct_out_end[r] = (r + 1) * chunk; }
                if (ag) { P.direct_in_start[r] = r * chunk; P.direct_in_end[r] = (r + 1) * chunk; }
            }
            std::vector<int64_t> cuts2 = {0, n};
            for (auto& sg : P.segs) { cuts2.push_back(sg.start); cuts2.push_back(sg.end); }
            if (!ar) for (int r = 0; r <= R; ++r) cuts2.push_back(r * chunk);
            std::sort(cuts2.begin(), cuts2.end());
            cuts2.erase(std::unique(cuts2.begin(), cuts2.end()), cuts2.end());
            bool valid = true;
            std::vector<ColInstr> prev_prog;
            const std::vector<ColSegment> base_segs = P.segs;
            size_t si = 0;
            for (size_t i = 0; i + 1 < cuts2.size() && valid; ++i) {
                const int64_t a = cuts2[i], b = cuts2[i + 1];
                if (a < 0 || b > n) continue;
                while (si < base_segs.size() && base_segs[si].end <= a) ++si;
                const ColSegment* under = (si < base_segs.size() && base_segs[si].start <= a && b <= base_segs[si].end) ? &base_segs[si] : nullptr;
                auto in_window = [&](int r) { return P.direct_in_start[r] <= a && b <= P.direct_in_end[r]; };
                auto out_window = [&](int r) { return P.direct_out_start[r] <= a && b <= P.direct_out_end[r]; };
                std::vector<ColInstr> prog;
                uint64_t written = 0;
                if (under)
                    for (size_t k = 0; k < raw_progs[si].size() && valid; ++k) {
                        ColInstr in = raw_progs[si][k];
                        if (in.a_src == SRC_MEM) valid = in.a_first ? in_window(in.peer) : out_window(in.peer);
                        if (valid && in.b_src == SRC_MEM) valid = in.b_first ? in_window(in.self) : out_window(in.self);
                        if (in.store && !out_window(in.self)) {
                            if (in.store == 1) valid = false;   // written outside the window and read back
                            in.store = 0;
                        }
                        if (in.store) written |= 1ull << in.self;
                        prog.push_back(in);
                    }
                for (int r = 0; r < R && valid; ++r)
                    if (out_window(r) && !(written >> r & 1)) {
                        if (!in_window(r)) { valid = false; break; }   // the reference would hand back stale buffer contents
                        ColInstr in{};
                        in.self = in.peer = (uint8_t)r; in.a_src = SRC_MEM; in.b_src = SRC_NONE;
                        in.a_first = 1; in.store = 2;
                        prog.push_back(in);
                    }
                if (!valid) break;
                // an instruction that neither stores nor feeds a later one can go
                while (!prog.empty() && !prog.back().store) prog.pop_back();
                if (prog.empty()) { prev_prog.clear(); continue; }
                auto same = [&](const std::vector<ColInstr>& x, const std::vector<ColInstr>& y) {
                    return x.size() == y.size() && std::memcmp(x.data(), y.data(), x.size() * sizeof(ColInstr)) == 0;
                };
                if (!P.direct_segs.empty() && P.direct_segs.back().end == a && same(prog, prev_prog)) {
                    P.direct_segs.back().end = b;
                    continue;
                }
                ColSegment d;
                d.start = a; d.end = b;
                d.prog_start = (int)P.col_instrs.size(); d.prog_len = (int)prog.size();
                prev_prog = prog;                      // compared before the finishing marks are added
                finish_column_program(P, d, prog);
                P.col_instrs.insert(P.col_instrs.end(), prog.begin(), prog.end());
                P.direct_segs.push_back(d);
            }
            if (!valid) P.direct_segs.clear();
            for (auto& seg : P.direct_segs)
                count_column_traffic(P, seg, es, &P.direct_load_bytes, &P.direct_store_bytes, &P.direct_slot_load_bytes, &P.direct_slot_store_bytes);
            plan_chains(P, P.direct_segs, &P.direct_chain_segs);
        }
    }
};

}  // namespace

Program link_program(const std::vector<const RankGraph*>& graphs, const LinkOptions& opt) {
    if (graphs.empty() || graphs.size() > (size_t)PCCL_HIP_MAX_VRANKS)
        throw Error{PCCL_ERR_INVALID, "number of virtual ranks must be 1.." + std::to_string(PCCL_HIP_MAX_VRANKS)};
    return Linker(graphs, opt).run();
}

}  // namespace pccl_hip
