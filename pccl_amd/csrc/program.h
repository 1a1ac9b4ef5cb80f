// Linked program: R per-rank graphs folded into one dependency graph of data ops, plus the two
// execution plans derived from it (column plan and stepwise plan).
#pragma once

#include <cstdint>
#include <string>
#include <vector>

#include "graph.h"

namespace pccl_hip {

struct LinkedOp {
    int rank = 0, channel = 0, graph_pos = 0, index = 0;
    bool is_reduce = false;
    int redop = PCCL_SUM;
    int peer = 0;
    int64_t off0 = 0, off1 = 0, off2 = 0, size = 0;
    int level = 0;
    std::vector<int> deps;  // indices into Program::ops (after ordering)

    int64_t dst_off() const { return is_reduce ? off2 : off1; }
    bool position_aligned() const { return is_reduce ? (off0 == off1 && off1 == off2) : (off0 == off1); }
};

// Operand sources of a column instruction.
enum : uint8_t { SRC_NONE = 0, SRC_MEM = 1, SRC_ACC = 2 };
// ColInstr::store: low two bits as documented there; STORE_LAST marks the last write of that rank
// in the program (its value must reach memory even when a later instruction reads it back).
enum : uint8_t { STORE_KIND = 3, STORE_LAST = 4 };

// One step of a segment's column program: acc = a (copy) or acc = a (op) b (reduce), then
// optionally mem[self] = acc.  a is the peer's value, b the own value.
struct ColInstr {
    uint8_t self;
    uint8_t peer;
    uint8_t a_src;   // SRC_MEM | SRC_ACC
    uint8_t b_src;   // SRC_NONE (copy) | SRC_MEM | SRC_ACC
    uint8_t redop;
    uint8_t store;   // & STORE_KIND: 0: the write is dead (overwritten before anything reads it from
                     // memory), 1: written and read back later by this program, 2: final value
                     // (streaming store); | STORE_LAST: no later instruction writes this rank
    uint8_t a_first; // 1: this load is the first access to (peer, position) in the program
    uint8_t b_first;
};
static_assert(sizeof(ColInstr) == 8, "ColInstr is read as one 8-byte word on the device");

struct ColSegment {
    int64_t start = 0, end = 0;  // element positions [start, end)
    int32_t prog_start = 0, prog_len = 0;
    int32_t pre_start = 0, pre_words = 0;  // words in Program::col_pre: the ranks this program reads by
                                           // first touch, 8 per word (one byte each, 0xFF = none), in
                                           // program order without repeats
    uint64_t bcast_mask = 0;               // ranks that receive the program's last value after its
                                           // last instruction (the tail of copies of one value)
};

// A segment whose column program is one chain: one accumulator takes the original values of the
// ranks in `srcs` one after another (acc = x[src 0]; acc = x[src k] (op) acc), and the final value
// is the only thing stored, to every rank of `store_mask`.  What the phased runner executes.
// Or, tree_depth = D > 0: the value is a perfectly balanced binary tree over 2^D ranks - srcs lists
// them leaf by leaf, left to right; leaves 2i and 2i + 1 are combined first, then those results in
// pairs, and so on (halving-doubling and binary-tree schedules under an operator whose rounding makes
// the shape matter).
struct ChainSegment {
    int64_t start = 0, end = 0;          // element positions [start, end)
    int32_t src_start = 0, n_src = 0;    // ranks in Program::chain_srcs, in the order they are combined
    int32_t redop = PCCL_SUM;
    int32_t tree_depth = 0;
    uint64_t store_mask = 0;
};

struct StepOpPlan {
    int first_item = 0, ntiles = 0, dep_start = 0, ndeps = 0;
    int lead = 0;   // elements between the item grid's anchor and the op's first element (< tile_elems)
};

// One semaphore a program touches: how often one execution notifies it and waits on it.  The counts a
// program leaves behind are (carried in) + notifies - waits, whatever order the ranks ran in.
struct SignalUse {
    int32_t rank = 0, id = 0;       // the semaphore: signal `id` of rank `rank`
    int32_t notifies = 0, waits = 0;
};

struct Program {
    int R = 0;
    int dtype = PCCL_F32;
    std::string collective_type;
    int64_t tensor_elems = 0;
    std::vector<LinkedOp> ops;  // topological order: (level, rank, channel, position)
    int num_all_ops = 0;
    int num_levels = 0;
    int residual_signals = 0;       // semaphores one execution leaves at another count than it found
    std::vector<SignalUse> signals; // every semaphore the program touches, ordered by (rank, id)
    int carried_waits = 0;          // waits that passed on a count carried in (LinkOptions::carried)
    int64_t buffer_elems = 0;
    int64_t algorithmic_bytes = 0;
    bool race_checked = false;    // the data-race check ran over every pair of conflicting accesses
    bool order_checked = false;   // the notify / wait pairing was checked for ambiguity (skipped above kClosureLimit ops)

    // column plan (valid when position_aligned)
    bool position_aligned = false;
    std::vector<ColSegment> segs;
    std::vector<ColInstr> col_instrs;
    std::vector<uint64_t> col_pre;
    int64_t column_load_bytes = 0, column_store_bytes = 0;   // with values re-read through memory
    int64_t slot_load_bytes = 0, slot_store_bytes = 0;       // with re-read values kept on chip
    // direct plan (staging fused into the program; valid when non-empty): covers [0, tensor_elems)
    std::vector<ColSegment> direct_segs;
    int64_t direct_load_bytes = 0, direct_store_bytes = 0;
    int64_t direct_slot_load_bytes = 0, direct_slot_store_bytes = 0;
    std::vector<int64_t> direct_in_start, direct_in_end, direct_out_start, direct_out_end;  // windows per rank

    // chain form of the two column plans: one entry per segment, or empty when some segment is not a
    // chain (values read back, results stored along the way, different values left in different ranks)
    std::vector<ChainSegment> chain_segs, direct_chain_segs;
    std::vector<uint8_t> chain_srcs;

    // gather plan of an alltoall graph (valid when non-empty): the staged call as direct copies from
    // the callers' input tensors to their output tensors, element units
    struct GatherCopy { int dst_rank, src_rank; int64_t dst_off, src_off, elems; };
    std::vector<GatherCopy> gather;

    // stepwise plan
    int64_t tile_elems = 0;
    std::vector<StepOpPlan> step_ops;
    std::vector<int32_t> step_deps;
    int64_t num_items = 0;
};

struct LinkOptions {
    bool check_races = true;
    bool conflict_deps = true;     // order data ops by memory conflicts instead of raw chain order
    int64_t step_tile_bytes = 0;   // bytes per work item of the stepwise plan; 0 = chosen from the program's size
    // Semaphore counts this execution finds, left by earlier executions on the same engine (the
    // reference clears its signal region only in Engine::resetSignals, csrc/engine_c.cc:576-593):
    // ((rank, id), count) for the counts above zero.  The first `count` waits on such a semaphore
    // pass without a notify of this execution and get no ordering from one.
    std::vector<std::pair<std::pair<int, int>, int>> carried;
};

// The semaphores the graphs touch, without linking them (registration order does not matter).
std::vector<SignalUse> signal_uses(const std::vector<const RankGraph*>& graphs);

// Throws Error (PCCL_ERR_LINK for deadlock, ambiguous signal pairing, races, bad ranks).
Program link_program(const std::vector<const RankGraph*>& graphs, const LinkOptions& opt);

}  // namespace pccl_hip
