// C ABI: host-only graph tools and the device executor context.
#include <dlfcn.h>
#include <hip/hip_runtime_api.h>

#include <cerrno>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <atomic>
#include <cstring>
#include <map>
#include <memory>
#include <mutex>
#include <string>
#include <vector>

#include "graph.h"
#include "kernels.h"
#include "program.h"

using namespace pccl_hip;

struct pccl_graph { RankGraph g; };
struct pccl_program { Program p; };

namespace {

thread_local std::string t_err;

int fail(int code, const std::string& msg) {
    t_err = msg;
    return code;
}

// Log lines on stderr, levels and the PCCL_LOG_LEVEL switch as in the reference
// (csrc/common/logging.cc:6-35, default WARN); stdout stays free for the caller's own output.
enum LogLevel { LOG_TRACE, LOG_DEBUG, LOG_INFO, LOG_WARN, LOG_ERROR, LOG_CRITICAL };

int log_threshold() {
    static const int level = [] {
        const char* v = std::getenv("PCCL_LOG_LEVEL");
        const std::string s = v ? v : "";
        const char* names[] = {"TRACE", "DEBUG", "INFO", "WARN", "ERROR", "CRITICAL"};
        for (int i = 0; i < 6; ++i)
            if (s == names[i]) return i;
        return (int)LOG_WARN;
    }();
    return level;
}

void log_line(int level, const std::string& msg) {
    if (level < log_threshold()) return;
    const char* tags[] = {"trace", "debug", "info", "warning", "error", "critical"};
    std::fprintf(stderr, "[pccl] [%s] %s\n", tags[level], msg.c_str());
}

template <class F>
int guarded(F&& f) {
    try {
        return f();
    } catch (const Error& e) {
        // the caller gets the message with the status code; the log repeats it only on request
        log_line(e.code == PCCL_ERR_HIP ? LOG_ERROR : LOG_INFO, "call failed (" + std::to_string(e.code) + "): " + e.msg);
        return fail(e.code, e.msg);
    } catch (const std::bad_alloc&) {
        return fail(PCCL_ERR_INVALID, "out of host memory");
    } catch (const std::exception& e) {
        return fail(PCCL_ERR_INVALID, e.what());
    }
}

#define HIP_TRY(expr)                                                                                   \
    do {                                                                                                \
        hipError_t e_ = (expr);                                                                         \
        if (e_ != hipSuccess) throw Error{PCCL_ERR_HIP, std::string(#expr) + ": " + hipGetErrorString(e_)}; \
    } while (0)

// Host-side ranges for a profiler's timeline, under the names of the reference's NVTX ranges
// (include/common/nvtx.h:7-16; engine_c.cc:468,485,489; cuda_device.cc:313,319).  The marker
// library is looked up at run time, the first time a context asks for ranges; without it (or
// without the option) a range costs one branch.
struct MarkerApi {
    int (*push)(const char*) = nullptr;
    int (*pop)() = nullptr;
};

const MarkerApi& marker_api() {
    static const MarkerApi api = [] {
        MarkerApi m;
        for (const char* lib : {"librocprofiler-sdk-roctx.so.1", "librocprofiler-sdk-roctx.so", "libroctx64.so.4", "libroctx64.so"}) {
            void* h = dlopen(lib, RTLD_NOW | RTLD_GLOBAL);
            if (!h) continue;
            m.push = (int (*)(const char*))dlsym(h, "roctxRangePushA");
            m.pop = (int (*)())dlsym(h, "roctxRangePop");
            if (m.push && m.pop) break;
            m = MarkerApi{};
        }
        return m;
    }();
    return api;
}

class TraceRange {
  public:
    TraceRange(bool wanted, const char* name) : on_(wanted && marker_api().push) { if (on_) marker_api().push(name); }
    ~TraceRange() { if (on_) marker_api().pop(); }
    TraceRange(const TraceRange&) = delete;
    TraceRange& operator=(const TraceRange&) = delete;
  private:
    bool on_;
};

void fill_info(const Program& p, pccl_program_info* out) {
    std::memset(out, 0, sizeof(*out));
    out->num_vranks = p.R;
    out->dtype = p.dtype;
    out->num_ops = p.num_all_ops;
    out->num_data_ops = (int)p.ops.size();
    out->num_levels = p.num_levels;
    out->position_aligned = p.position_aligned;
    out->num_segments = (int)p.segs.size();
    out->residual_signals = p.residual_signals;
    out->buffer_elems = p.buffer_elems;
    out->algorithmic_bytes = p.algorithmic_bytes;
    out->column_load_bytes = p.column_load_bytes;
    out->column_store_bytes = p.column_store_bytes;
    out->num_items = (int)p.num_items;
    out->num_gather_copies = (int)p.gather.size();
    out->staged_load_bytes = p.direct_load_bytes;
    out->staged_store_bytes = p.direct_store_bytes;
    out->race_checked = p.race_checked;
    out->order_checked = p.order_checked;
    out->chain_segments = (int)p.chain_segs.size();
    out->staged_chain_segments = (int)p.direct_chain_segs.size();
}

// What a reader of the log should know about a linked program, said once at link time (WARN, the
// default threshold).  The reference keeps its counting semaphores across executions and across
// operations (zeroed only by resetSignals, csrc/engine_c.cc:576-593; a wait passes on any count
// above zero and takes one, csrc/plugins/cuda/cuda_executor.cu:425-445), and so does an engine
// here: a notify nobody awaits is found by the next execution that waits on that semaphore.
void warn_about(const Program& p, const std::string& what, bool races_wanted) {
    if (p.residual_signals != 0)
        log_line(LOG_WARN, what + ": one execution leaves " + std::to_string(p.residual_signals) + " semaphore(s) at another count than it "
                               "found them (notifies and waits do not balance); the counts are carried into the next execution of any "
                               "operation on this engine, as in the reference, until reset_signals");
    if (p.carried_waits != 0)
        log_line(LOG_INFO, what + ": " + std::to_string(p.carried_waits) + " wait(s) pass on counts that earlier executions left behind");
    if (!p.order_checked)
        log_line(LOG_WARN, what + ": " + std::to_string(p.num_all_ops) + " ops are too many for the notify/wait ambiguity check and the "
                               "data-race check; the pairing of one valid execution order is used unverified");
    else if (races_wanted && !p.race_checked && p.ops.size() > 1)
        log_line(LOG_WARN, what + ": the data-race check gave up (too many overlapping accesses); conflicting accesses are not verified to be ordered");
}

}  // namespace

extern "C" {

const char* pccl_hip_last_error(void) { return t_err.c_str(); }
const char* pccl_hip_version(void) { return "pccl-hip 0.1 (gfx950)"; }

// ------------------------------------------------------------------------------- graph tools

int pccl_graph_load_file(const char* path, pccl_graph** out) {
    return guarded([&] {
        if (!path || !out) return fail(PCCL_ERR_INVALID, "null argument");
        auto g = std::make_unique<pccl_graph>();
        g->g = load_graph_file(path);
        *out = g.release();
        return 0;
    });
}

int pccl_graph_load_json(const char* text, size_t len, pccl_graph** out) {
    return guarded([&] {
        if (!text || !out) return fail(PCCL_ERR_INVALID, "null argument");
        auto g = std::make_unique<pccl_graph>();
        g->g = load_graph_json(text, len);
        *out = g.release();
        return 0;
    });
}

int pccl_graph_from_triggers(const pccl_trigger* triggers, const pccl_primitive_meta* meta, int n,
                             const char* collective_type, pccl_graph** out) {
    return guarded([&] {
        if (!out) return fail(PCCL_ERR_INVALID, "null argument");
        auto g = std::make_unique<pccl_graph>();
        g->g = graph_from_triggers(triggers, meta, n, collective_type);
        *out = g.release();
        return 0;
    });
}

void pccl_graph_free(pccl_graph* g) { delete g; }
int pccl_graph_num_ops(const pccl_graph* g) { return g ? (int)g->g.ops.size() : PCCL_ERR_INVALID; }
int pccl_graph_dtype(const pccl_graph* g) { return g ? g->g.dtype : PCCL_ERR_INVALID; }
int64_t pccl_graph_tensor_elems(const pccl_graph* g) { return g ? g->g.tensor_elems : 0; }
const char* pccl_graph_collective_type(const pccl_graph* g) { return g ? g->g.collective_type.c_str() : ""; }

// How many of `have` records fit into a caller's array of `cap` (a negative cap holds none).
static size_t fits(int cap, size_t have) { return cap <= 0 ? 0 : std::min<size_t>((size_t)cap, have); }

int pccl_graph_get_triggers(const pccl_graph* g, pccl_trigger* out, int cap) {
    return guarded([&] {
        if (!g || !out) return fail(PCCL_ERR_INVALID, "null argument");
        std::vector<pccl_trigger> t;
        graph_to_triggers(g->g, &t, nullptr);
        std::memcpy(out, t.data(), sizeof(pccl_trigger) * fits(cap, t.size()));
        return (int)t.size();
    });
}

int pccl_graph_get_meta(const pccl_graph* g, pccl_primitive_meta* out, int cap) {
    return guarded([&] {
        if (!g || !out) return fail(PCCL_ERR_INVALID, "null argument");
        std::vector<pccl_primitive_meta> m;
        graph_to_triggers(g->g, nullptr, &m);
        std::memcpy(out, m.data(), sizeof(pccl_primitive_meta) * fits(cap, m.size()));
        return (int)m.size();
    });
}

int pccl_graph_fused_steps(const pccl_graph* g, pccl_fused_step* steps, int cap, int* channel_offsets,
                           int* num_channels) {
    return guarded([&] {
        if (!g) return fail(PCCL_ERR_INVALID, "null argument");
        std::vector<pccl_fused_step> s;
        std::vector<int> off;
        if (!build_fused_steps(g->g, &s, &off))
            return fail(PCCL_ERR_UNSUPPORTED, "graph is not a set of per-channel linear chains of at most 128 steps");
        if (steps) std::memcpy(steps, s.data(), sizeof(pccl_fused_step) * fits(cap, s.size()));
        if (channel_offsets)
            for (size_t i = 0; i < off.size() && i <= PCCL_HIP_MAX_CHANNELS; ++i) channel_offsets[i] = off[i];
        if (num_channels) *num_channels = (int)off.size() - 1;
        return (int)s.size();
    });
}

int pccl_program_link(const pccl_graph* const* graphs, int num_vranks, pccl_program** out) {
    return guarded([&] {
        if (!graphs || !out) return fail(PCCL_ERR_INVALID, "null argument");
        std::vector<const RankGraph*> gs;
        for (int r = 0; r < num_vranks; ++r) gs.push_back(graphs[r] ? &graphs[r]->g : nullptr);
        auto p = std::make_unique<pccl_program>();
        p->p = link_program(gs, LinkOptions{});
        warn_about(p->p, "linked program", true);
        *out = p.release();
        return 0;
    });
}

int pccl_program_link_carried(const pccl_graph* const* graphs, int num_vranks, const int32_t* carried, int num_carried,
                              pccl_program** out) {
    return guarded([&] {
        if (!graphs || !out || (num_carried > 0 && !carried) || num_carried < 0) return fail(PCCL_ERR_INVALID, "null argument");
        std::vector<const RankGraph*> gs;
        for (int r = 0; r < num_vranks; ++r) gs.push_back(graphs[r] ? &graphs[r]->g : nullptr);
        LinkOptions opt;
        for (int i = 0; i < num_carried; ++i) {
            const int32_t* c = carried + 3 * (size_t)i;
            if (c[0] < 0 || c[0] >= num_vranks || c[2] < 0)
                return fail(PCCL_ERR_INVALID, "carried count " + std::to_string(i) + ": rank " + std::to_string(c[0]) + ", count " + std::to_string(c[2]));
            opt.carried.push_back({{(int)c[0], (int)c[1]}, (int)c[2]});
        }
        auto p = std::make_unique<pccl_program>();
        p->p = link_program(gs, opt);
        warn_about(p->p, "linked program", true);
        *out = p.release();
        return 0;
    });
}

int pccl_program_get_signals(const pccl_program* p, int32_t* out, int cap) {
    if (!p || (!out && cap > 0)) return fail(PCCL_ERR_INVALID, "null argument");
    const std::vector<SignalUse>& u = p->p.signals;
    for (size_t i = 0; i < u.size() && (int)i < cap; ++i) {
        out[4 * i] = u[i].rank; out[4 * i + 1] = u[i].id; out[4 * i + 2] = u[i].notifies; out[4 * i + 3] = u[i].waits;
    }
    return (int)u.size();
}

void pccl_program_free(pccl_program* p) { delete p; }

int pccl_program_get_info(const pccl_program* p, pccl_program_info* out) {
    if (!p || !out) return fail(PCCL_ERR_INVALID, "null argument");
    fill_info(p->p, out);
    return 0;
}

int pccl_program_get_ops(const pccl_program* p, pccl_linked_op* out, int cap) {
    if (!p || !out) return fail(PCCL_ERR_INVALID, "null argument");
    const int n = (int)fits(cap, p->p.ops.size());
    for (int k = 0; k < n; ++k) {
        const LinkedOp& L = p->p.ops[k];
        pccl_linked_op& o = out[k];
        std::memset(&o, 0, sizeof(o));
        o.rank = L.rank; o.channel = L.channel; o.op_index = L.index; o.is_reduce = L.is_reduce;
        o.redop = L.redop; o.peer_rank = L.peer; o.level = L.level; o.num_deps = (int)L.deps.size();
        o.offset_0 = L.off0; o.offset_1 = L.off1; o.offset_2 = L.off2; o.size = L.size;
        for (size_t d = 0; d < L.deps.size() && d < 8; ++d) o.deps[d] = L.deps[d];
    }
    return (int)p->p.ops.size();
}

int pccl_program_get_column(const pccl_program* p, int which,
                            pccl_column_segment* segs, int seg_cap, int* n_segs,
                            uint64_t* instrs, int instr_cap, int* n_instrs,
                            uint64_t* pre, int pre_cap, int* n_pre,
                            int64_t* in_window, int64_t* out_window) {
    if (!p || !n_segs || !n_instrs || !n_pre) return fail(PCCL_ERR_INVALID, "null argument");
    if (which != 0 && which != 1) return fail(PCCL_ERR_INVALID, "which must be 0 (in place) or 1 (staged)");
    const Program& P = p->p;
    const std::vector<ColSegment>& src = which ? P.direct_segs : P.segs;
    *n_segs = (int)src.size(); *n_instrs = (int)P.col_instrs.size(); *n_pre = (int)P.col_pre.size();
    for (int i = 0; segs && i < seg_cap && i < (int)src.size(); ++i) {
        segs[i].start = src[i].start; segs[i].end = src[i].end;
        segs[i].prog_start = src[i].prog_start; segs[i].prog_len = src[i].prog_len;
        segs[i].pre_start = src[i].pre_start; segs[i].pre_words = src[i].pre_words;
        segs[i].bcast_mask = src[i].bcast_mask;
    }
    static_assert(sizeof(ColInstr) == sizeof(uint64_t), "instruction words");
    if (instrs) std::memcpy(instrs, P.col_instrs.data(), sizeof(uint64_t) * fits(instr_cap, P.col_instrs.size()));
    if (pre) std::memcpy(pre, P.col_pre.data(), sizeof(uint64_t) * fits(pre_cap, P.col_pre.size()));
    if (which == 1 && !P.direct_segs.empty())
        for (int r = 0; r < P.R; ++r) {
            if (in_window) { in_window[2 * r] = P.direct_in_start[r]; in_window[2 * r + 1] = P.direct_in_end[r]; }
            if (out_window) { out_window[2 * r] = P.direct_out_start[r]; out_window[2 * r + 1] = P.direct_out_end[r]; }
        }
    return 0;
}

}  // extern "C"

// ------------------------------------------------------------------------------- device context

namespace {

struct DevBuf {
    void* p = nullptr;
    size_t bytes = 0;
    void release() { if (p) { (void)hipFree(p); p = nullptr; bytes = 0; } }
    void upload(const void* src, size_t n) {
        release();
        if (n == 0) return;
        HIP_TRY(hipMalloc(&p, n));
        bytes = n;
        HIP_TRY(hipMemcpy(p, src, n, hipMemcpyHostToDevice));
    }
};

struct OpEntry {
    std::vector<std::unique_ptr<RankGraph>> graphs;
    bool linked = false;
    Program prog;
    DevBuf gather;                        // gather plan of an alltoall graph (DevGatherCopy records)
    int64_t gather_tiles = 0;
    int gather_copy_tiles = 0;            // > 0: every copy of the gather plan has this many tiles
    // Linking has a host half (the program and the tables derived from it; no HIP call) and a device
    // half (the tables uploaded: allocations and copies).  Inspection needs the first only; the
    // second happens at the first execution, and not on a stream that is being captured.
    bool host_linked = false;
    bool uses_scanned = false;
    std::vector<SignalUse> sig_uses;      // the semaphores the graphs touch (depends on the graphs only)
    std::vector<int> link_carried;        // per sig_uses entry: the carried count the current link was made for
    struct HostTables {
        std::vector<DevColSegment> segs, direct_segs;
        std::vector<DevChainSegment> chain_segs, direct_chain_segs;   // phased runner (empty: the plan is not a chain plan)
        std::vector<int32_t> chain_srcs;                               // one word per source rank, padded to whole 8-byte words
        std::vector<DevGatherCopy> gather;
        std::vector<DevStepOp> step_ops;
        std::vector<int32_t> item_op;
        std::vector<int32_t> step_deps_padded;   // the dependency lists padded to whole 8-byte words
    } host;
    DevBuf segs, direct_segs, instrs, pre, step_ops, step_deps, item_op, state;
    DevBuf chain_segs, direct_chain_segs, chain_srcs, phase_sync;
    int64_t chain_chunks = 0, direct_chain_chunks = 0;   // phased runner: chunks of the two chain plans
    int chain_seg_chunks = 0, direct_chain_seg_chunks = 0;   // > 0: every segment has this many chunks
    int chain_tree = 0, direct_chain_tree = 0;               // the plan holds balanced trees: the shape it runs on (0: none)
    bool chain_whole = false, direct_chain_whole = false;    // every chunk of the plan lies inside its segment (no cut chunks)
    bool chain_alike = false, direct_chain_alike = false;    // the segments are adjacent in memory, with the same number of sources, operator
                                                             // and store mask, their source lists one after the other
    int64_t total_tiles = 0, direct_tiles = 0;
    int seg_tiles = 0, direct_seg_tiles = 0;   // > 0: every segment of the plan has this many tiles
    int vecs_per_thread = 0;
    int slot_threads = 0;
    int slot_vecs = 1;                    // slot runner: vectors per thread
    int slot_lds_bytes = 0;               // slot runner: dynamic LDS per workgroup
    hipEvent_t ev0 = nullptr, ev1 = nullptr;
    bool timed = false;
    bool ran_persistent = false;          // a persistent launch has not been checked for stalls yet
    bool ran_static = false;              // the same for a launch in the static workspace
    bool stale_replay = false;            // a recorded launch of this operation was replayed on foreign tables; its next sync says so
    uint64_t generation = 0;              // which host link these tables come from (never reused in the process)
    int epoch = 0;                        // persistent runner: launches so far
    std::vector<int> level_item_begin;    // work-list index where each dependency level starts (+ end)
    // Level runner: the launches of one execution captured as a HIP graph, per set of rank
    // pointers (kernel arguments are frozen at capture time).  A handful are kept.
    struct LevelGraph { std::vector<char*> key; hipGraph_t graph = nullptr; hipGraphExec_t exec = nullptr; uint64_t used = 0; };
    std::vector<LevelGraph> level_graphs;
    uint64_t graph_clock = 0;
    bool graph_failed = false;            // capture did not work once: launch level by level from then on
    void drop_graphs() {
        for (auto& g : level_graphs) {
            if (g.exec) (void)hipGraphExecDestroy(g.exec);
            if (g.graph) (void)hipGraphDestroy(g.graph);
        }
        level_graphs.clear();
    }
    void release() {
        drop_graphs();
        graph_failed = false;
        gather.release(); gather_tiles = 0;
        segs.release(); direct_segs.release(); instrs.release(); pre.release(); step_ops.release(); step_deps.release();
        item_op.release(); state.release();
        chain_segs.release(); direct_chain_segs.release(); chain_srcs.release(); phase_sync.release();
        if (ev0) (void)hipEventDestroy(ev0);
        if (ev1) (void)hipEventDestroy(ev1);
        ev0 = ev1 = nullptr;
        linked = false; timed = false;
        host_linked = false; host = HostTables{};
    }
};

enum class Mode { Auto, Column, Stepwise, Persistent };
constexpr size_t kMaxSlotLdsBytes = 160 * 1024;   // LDS of one gfx950 CU

// Shape of a slot-runner workgroup for R ranks under the given option values (0 = automatic):
// threads x vectors per thread (a tile is that many 16-byte vectors of every rank) and the LDS its
// slots need.  The one place that decides it: linking uses it, and set_option checks a new value
// against it, so that a combination the LDS cannot hold is refused where it is asked for.
// Measured on MI355X, same box and call: 8 ranks x 512 MiB bf16 ring 256 x 1 (five per CU) 1.43 ms,
// 256 x 2 (two per CU, 8 KiB of every rank per tile) 1.39; 32-rank tree 64 x 1 1.19 ms, 128 x 1
// 1.12; 16 ranks the same from 128 to 512 threads.  One workgroup per CU with larger tiles loses:
// the program's arithmetic is then not overlapped with anything.
struct SlotShape { int threads, vecs; size_t need; };
SlotShape slot_shape(int R, int slot_threads, int slot_vecs, bool slot_direct) {
    SlotShape sh;
    sh.threads = R <= 16 ? 256 : R <= 32 ? 128 : 64;
    sh.vecs = R > 4 && R <= 8 ? 2 : 1;
    if (slot_threads > 0) { sh.threads = slot_threads; if (slot_vecs == 0) sh.vecs = 1; }
    if (slot_vecs > 0) sh.vecs = slot_vecs;
    if (!slot_direct) sh.vecs = 1;   // fetching through registers: one vector per thread
    sh.need = (size_t)R * sh.vecs * sh.threads * 16;
    return sh;
}
// Empty if the shape can be launched, else why not.
std::string slot_shape_error(int R, const SlotShape& sh) {
    if (sh.threads * sh.vecs > 1024) return "slot runner: slot_threads x slot_vecs may not exceed 1024 (" + std::to_string(sh.threads) + " x " + std::to_string(sh.vecs) + ")";
    if (sh.need > kMaxSlotLdsBytes)
        return "slot runner: " + std::to_string(R) + " ranks x " + std::to_string(sh.vecs) + " vectors x " + std::to_string(sh.threads) +
               " threads x 16 bytes exceed the " + std::to_string(kMaxSlotLdsBytes >> 10) + " KiB of LDS a workgroup may use";
    return "";
}

}  // namespace

struct pccl_hip_ctx {
    int device = 0;
    int R = 0;
    std::mutex mu;
    std::map<std::string, OpEntry> ops;
    std::vector<char*> bufs;   // engine-owned rank buffers (staged execution)
    size_t buf_bytes = 0;
    Mode mode = Mode::Auto;
    int num_blocks = 0;
    int vecs_per_thread = 1;
    bool check_races = true;
    bool timing = false;
    bool trace_ranges = false;            // emit profiler ranges around the stages of a call
    bool lds_slots = true;                // column runner keeps re-read values in LDS slots
    int slot_threads = 0;                 // slot runner workgroup size (0: chosen from the rank count)
    int slot_vecs = 0;                    // slot runner vectors per thread (0: chosen from the rank count)
    int slot_lds_kib = 0;                 // slot runner: least dynamic LDS a workgroup asks for (0: chosen), which bounds the workgroups per CU
    bool slot_direct = true;              // slot runner fetches first touches straight into LDS
    int slot_store_waves = -1;            // slot runner: broadcast tail through LDS, whole tiles of a rank stored by one wave
                                          // (1), every wave a slice of every rank (0), or chosen from the plan's traffic (-1)
    int phased = -1;                      // chain plans on the phased runner (whole chip reads, then writes): 1 whenever the
                                          // plan is a chain plan, 0 never, -1 when it is and the tensors are large enough
    int phased_exchange = -1;             // 256 x 32 shapes: the sums change hands through LDS between read and write phase (-1 chosen, 0, 1)
    int phased_sweeps = -1;               // sweeps read before their sums are written: 1, 2 (512 x 16 only), -1: 2 for plans that mostly read
    int phased_linear = -1;               // chunks of 128 neighbouring workgroups interleaved slab by slab where the plan allows it (-1 chosen, 0, 1)
    int phased_shape = -1;                // its workgroup: 0 = 512 threads x 16 vectors, 1 = 256 x 32 (a wave's vectors contiguous), -1 chosen
    bool phased_barriers = true;          // its workgroups meet between the phases (0: they run free, for comparison)
    int phased_timeout_us = 1000;         // how long a workgroup waits at a meeting point before the launch goes on unsynchronised
    bool level_graph = false;             // level runner replays its launches as one HIP graph (measured:
                                          // no faster than launching level by level, so off by default)
    hipStream_t capture_stream = nullptr; // private stream the level launches are captured on
    int64_t step_tile_bytes = 0;   // work item of the level and persistent runners; 0 = automatic, 32 KiB for large programs (persistent, headline graph: 3.91 ms at 8 KiB, 3.16 at 16, 3.10 at 32, 3.35 at 64; sizes that do not divide the ops are slower)
    bool fuse_staging = true;             // run staged calls on the caller's tensors when possible
    int wait_timeout_ms = 2000;           // a persistent launch gives up on a dependency after this long
    int32_t host_epoch_limit = kHostEpochLimit;   // persistent runner: launch number at which the host clears the flags and restarts
    int32_t graph_epoch_limit = kGraphEpochLimit; // the same for the device-side counter of recorded launches
    hipStream_t last_stream = nullptr;
    // Counting semaphores above zero, (rank, id) -> count: what executions so far have left behind.
    // One state per engine, shared by all operations, cleared by pccl_hip_reset_signals - the
    // reference's signal region (csrc/engine_c.cc:131-146, 576-593).  Updated when an execution is
    // issued: executions are ordered by the streams they are issued to, as the caller orders them.
    std::map<std::pair<int, int>, int> signals;
};

namespace {

bool is_capturing(hipStream_t s) {
    hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
    return hipStreamIsCapturing(s, &cap) == hipSuccess && cap != hipStreamCaptureStatusNone;
}

// Set-up work (linking, table uploads, growing the rank buffers) allocates and synchronises, which
// would invalidate a capture in progress on the caller's stream: refuse instead.
void refuse_setup_under_capture(hipStream_t s, const char* what) {
    if (is_capturing(s))
        throw Error{PCCL_ERR_INVALID, std::string("the stream is capturing and this call would have to ") + what +
                                          ": execute the operation once outside the capture first"};
}

void ensure_buffers(pccl_hip_ctx* ctx, size_t bytes, hipStream_t stream) {
    if (bytes <= ctx->buf_bytes) return;
    refuse_setup_under_capture(stream, "grow the engine's rank buffers");
    // every registered op aliases the same rank buffers (as in the reference, engine_c.cc:191-196)
    HIP_TRY(hipDeviceSynchronize());
    for (char*& b : ctx->bufs) { if (b) (void)hipFree(b); b = nullptr; }
    ctx->buf_bytes = 0;
    size_t rounded = (bytes + 4095) & ~(size_t)4095;
    for (int r = 0; r < ctx->R; ++r) {
        void* p = nullptr;
        HIP_TRY(hipMalloc(&p, rounded));
        ctx->bufs[r] = (char*)p;
    }
    ctx->buf_bytes = rounded;
}

// The counts an execution of `e` would find now on the semaphores it touches, one per entry of
// e.sig_uses, cut off at the number of waits it has there (a higher count changes nothing for it).
std::vector<int> carried_now(pccl_hip_ctx* ctx, OpEntry& e) {
    if (!e.uses_scanned) {
        std::vector<const RankGraph*> gs;
        for (int r = 0; r < ctx->R; ++r) gs.push_back(r < (int)e.graphs.size() ? e.graphs[r].get() : nullptr);
        e.sig_uses = signal_uses(gs);
        e.uses_scanned = true;
    }
    std::vector<int> out;
    out.reserve(e.sig_uses.size());
    for (const SignalUse& u : e.sig_uses) {
        auto it = ctx->signals.find(std::make_pair((int)u.rank, (int)u.id));
        out.push_back(it == ctx->signals.end() ? 0 : std::min(it->second, (int)u.waits));
    }
    return out;
}

// Before an execution or an inspection of `e`: its link has to be the one for the counts its
// semaphores hold now.  A program whose waits find other counts than its link assumed pairs its
// notifies and waits differently (and may deadlock or race where it did not), so it is linked again;
// operations whose notifies and waits balance, on semaphores nobody left counts on - every schedule
// template - never come here twice.
void refresh_link(pccl_hip_ctx* ctx, OpEntry& e, hipStream_t s, bool executing, bool may_free_device = true) {
    const std::vector<int> now = carried_now(ctx, e);
    bool moves = false, carried = false;
    for (size_t i = 0; i < now.size(); ++i) {
        moves = moves || e.sig_uses[i].notifies != e.sig_uses[i].waits;
        carried = carried || now[i] > 0;
    }
    if (executing && (moves || carried) && is_capturing(s))
        throw Error{PCCL_ERR_INVALID, "the stream is capturing and this operation's semaphores carry counts from one execution to the next "
                                      "(its notifies and waits do not balance, or an earlier execution left counts on them): a recorded launch "
                                      "could not follow them.  Execute it outside the capture, or call reset_signals first if the counts are not wanted"};
    if ((e.host_linked || e.linked) && now != e.link_carried) {
        if (e.linked) {
            if (!may_free_device)
                throw Error{PCCL_ERR_INVALID, "the semaphore counts this operation finds have changed since it was linked and its plan tables on the "
                                              "device would have to be replaced, which this entry point may not do (it frees nothing): execute the "
                                              "operation once through pccl_hip_execute_inplace, or call reset_signals"};
            HIP_TRY(hipDeviceSynchronize());
        }
        e.release();
    }
}

// An execution of `e` has been issued: its notifies and waits are now part of the engine's state.
void commit_signals(pccl_hip_ctx* ctx, const OpEntry& e) {
    for (const SignalUse& u : e.sig_uses) {
        const int d = u.notifies - u.waits;
        if (d == 0) continue;
        const auto key = std::make_pair((int)u.rank, (int)u.id);
        int& c = ctx->signals[key];
        c += d;
        if (c <= 0) ctx->signals.erase(key);     // never below zero: the link would have reported a deadlock
    }
}

// Host half of linking: the program, the shape of the slot runner's workgroups, the tables as the
// kernels read them.  No HIP call.
void link_host(pccl_hip_ctx* ctx, OpEntry& e) {
    if (e.host_linked) return;
    e.host = OpEntry::HostTables{};
    std::vector<const RankGraph*> gs;
    for (int r = 0; r < ctx->R; ++r) gs.push_back(e.graphs[r].get());
    LinkOptions opt;
    opt.check_races = ctx->check_races;
    opt.step_tile_bytes = ctx->step_tile_bytes;
    const std::vector<int> carried = carried_now(ctx, e);
    for (size_t i = 0; i < carried.size(); ++i)
        if (carried[i] > 0) opt.carried.push_back({{(int)e.sig_uses[i].rank, (int)e.sig_uses[i].id}, carried[i]});
    e.link_carried = carried;
    e.prog = link_program(gs, opt);
    const Program& P = e.prog;
    const int es = elem_size(P.dtype);
    const int ve = 16 / es;
    e.vecs_per_thread = ctx->vecs_per_thread;

    // column plans (in place, and direct = staging fused into the program)
    if (P.position_aligned) {
        // The slot runner is the default.  Exception: a program that never reads a value back (every memory operand a first touch,
        // every live store final - the ring's chains) moves the same bytes under the register
        // runner, which needs no LDS; beyond 16 ranks the slots leave room for so few waves that it
        // wins (32-rank bf16 ring 0.99 -> 0.80 ms, 64-rank f32 ring 2.57 -> 1.62 ms; at 16 ranks
        // and below the slot runner's parallel fetch is still ahead).
        bool reads_back = false;
        for (const ColInstr& in : P.col_instrs)
            if ((in.a_src == SRC_MEM && !in.a_first) || (in.b_src == SRC_MEM && !in.b_first) || (in.store & STORE_KIND) == 1) reads_back = true;
        e.slot_threads = 0; e.slot_vecs = 1; e.slot_lds_bytes = 0;
        // Plans that mostly write (an allgather: one chunk in, R out; both the in-place and the staged
        // form) want larger workgroups whose waves each store whole tiles of a rank.  Measured on
        // MI355X, fp16 ring allgather as a staged call, fraction of the 8 TB/s: 32 ranks x 8 / 24 /
        // 96 MiB on the slot runner with 256 threads 0.715 / 0.778 / 0.670 against 0.694 / 0.715 /
        // 0.650 for the register runner; 8 ranks x 256 / 512 MiB with 1024 threads x 1 vector 0.752 /
        // 0.759 against 0.735 / 0.740 for 256 x 2 - below that size the smaller tiles win (128 MiB
        // 0.729 against 0.752, 32 MiB 0.64 against 0.70); 16 ranks x 64 / 256 MiB with 512 threads 0.723-0.732 /
        // 0.738-0.741 against 0.702 / 0.706-0.710 for 256, and 0.70 against 0.80 at 16 MiB.
        const bool mostly_writes = P.slot_store_bytes >= 4 * P.slot_load_bytes && P.slot_load_bytes > 0 &&
                                   (P.direct_segs.empty() || P.direct_slot_store_bytes >= 4 * P.direct_slot_load_bytes);
        const bool automatic = ctx->slot_threads == 0 && ctx->slot_vecs == 0 && ctx->slot_direct;
        const int64_t rank_bytes = P.tensor_elems * elem_size(P.dtype);
        if (ctx->lds_slots && (ctx->slot_threads > 0 || reads_back || ctx->R <= 16 || (mostly_writes && ctx->R <= 32))) {
            const int R = ctx->R;
            SlotShape sh = slot_shape(R, ctx->slot_threads, ctx->slot_vecs, ctx->slot_direct);
            if (automatic && mostly_writes) {
                if (R > 16) sh = slot_shape(R, 256, 1, true);
                else if (R > 4 && R <= 8 && rank_bytes >= ((int64_t)256 << 20)) sh = slot_shape(R, 1024, 1, true);
                else if (R > 8 && rank_bytes >= ((int64_t)64 << 20)) sh = slot_shape(R, 512, 1, true);
            }
            const std::string why = slot_shape_error(R, sh);
            if (!why.empty()) throw Error{PCCL_ERR_INVALID, why};
            const int threads = sh.threads, vecs = sh.vecs;
            const size_t need = sh.need;
            const int lds_kib = ctx->slot_lds_kib;
            e.slot_threads = threads; e.slot_vecs = vecs;
            e.slot_lds_bytes = (int)std::min<size_t>(std::max<size_t>(need, (size_t)lds_kib << 10), kMaxSlotLdsBytes);
        }
        const int64_t tile_v = e.slot_threads > 0 ? (int64_t)e.slot_threads * e.slot_vecs : 256 * (int64_t)e.vecs_per_thread;
        auto device_segments = [&](const std::vector<ColSegment>& segs, int64_t* total, int* uniform) {
            std::vector<DevColSegment> ds(segs.size());
            int64_t tiles = 0;
            for (size_t i = 0; i < segs.size(); ++i) {
                const ColSegment& s = segs[i];
                DevColSegment& d = ds[i];
                d.start = s.start; d.end = s.end;
                d.first_vec = s.start / ve;
                int64_t last_vec = (s.end - 1) / ve;
                d.first_tile = tiles;
                tiles += (last_vec - d.first_vec + 1 + tile_v - 1) / tile_v;
                d.prog_start = s.prog_start; d.prog_len = s.prog_len;
                d.pre_start = s.pre_start; d.pre_words = s.pre_words;
                d.streaming = 1; d.pad_ = 0; d.bcast_mask = s.bcast_mask;
                d.pre_mask = 0;
                for (int w = 0; w < s.pre_words; ++w)
                    for (int j = 0; j < 8; ++j) {
                        const unsigned r = (unsigned)(P.col_pre[s.pre_start + w] >> (8 * j) & 0xFF);
                        if (r != 0xFF) d.pre_mask |= 1ull << r;
                    }
                for (int k = 0; k < s.prog_len; ++k) {
                    const ColInstr& in = P.col_instrs[s.prog_start + k];
                    if ((in.a_src == SRC_MEM && !in.a_first) || (in.b_src == SRC_MEM && !in.b_first) || (in.store & STORE_KIND) == 1) d.streaming = 0;
                }
            }
            *total = tiles;
            // all segments the same number of tiles?  (the kernels then compute the segment of a tile)
            const int64_t per = ds.size() > 1 ? ds[1].first_tile : tiles;
            bool same = per > 0 && tiles == per * (int64_t)ds.size() && tiles < ((int64_t)1 << 32) && per <= INT32_MAX;
            for (size_t i = 0; i < ds.size() && same; ++i) same = ds[i].first_tile == (int64_t)i * per;
            *uniform = same ? (int)per : 0;
            return ds;
        };
        e.host.segs = device_segments(P.segs, &e.total_tiles, &e.seg_tiles);
        if (!P.direct_segs.empty()) e.host.direct_segs = device_segments(P.direct_segs, &e.direct_tiles, &e.direct_seg_tiles);
        // chain plans for the phased runner (both of its workgroup shapes take chunks of the same size)
        static_assert(phased_chunk_vecs(0) == phased_chunk_vecs(1) && phased_chunk_vecs(0) == phased_chunk_vecs(2), "one chunk table serves all shapes");
        auto chain_segments = [&](const std::vector<ChainSegment>& segs, int64_t* total, int* uniform, int* tree_shape, bool* all_whole, bool* alike) {
            std::vector<DevChainSegment> ds(segs.size());
            int64_t chunks = 0;
            int depth = 0;
            for (const ChainSegment& c : segs) depth = std::max(depth, c.tree_depth);
            // a plan with balanced trees runs on the shape that has the code for them (not built for the
            // 8-bit floats, whose arithmetic leaves no registers for it: those stay with the slot runner)
            *tree_shape = depth == 0 ? 0 : 2;
            *all_whole = !segs.empty();
            *alike = !segs.empty() && depth == 0;
            for (size_t i = 1; i < segs.size() && *alike; ++i)
                *alike = segs[i].n_src == segs[0].n_src && segs[i].redop == segs[0].redop && segs[i].store_mask == segs[0].store_mask &&
                         segs[i].src_start == segs[0].src_start + (int)i * segs[0].n_src && segs[i].start == segs[i - 1].end;
            if (depth > 0 && (P.dtype == PCCL_F8E4M3 || P.dtype == PCCL_F8E5M2)) { *total = 0; *uniform = 0; *all_whole = false; return std::vector<DevChainSegment>(); }
            const int64_t chunk_v = phased_chunk_vecs(*tree_shape);
            for (size_t i = 0; i < segs.size(); ++i) {
                const ChainSegment& c = segs[i];
                DevChainSegment& d = ds[i];
                d.start = c.start; d.end = c.end;
                d.first_vec = c.start / ve;
                const int64_t last_vec = (c.end - 1) / ve;
                d.first_chunk = chunks;
                chunks += (last_vec - d.first_vec + 1 + chunk_v - 1) / chunk_v;
                if (c.start % ve || (c.end - c.start) % (chunk_v * ve)) *all_whole = false;
                d.src_start = c.src_start; d.n_src = c.n_src; d.redop = c.redop; d.tree_depth = c.tree_depth; d.store_mask = c.store_mask;
            }
            *total = chunks;
            const int64_t per = ds.size() > 1 ? ds[1].first_chunk : chunks;
            bool same = per > 0 && chunks == per * (int64_t)ds.size() && chunks < ((int64_t)1 << 32) && per <= INT32_MAX;
            for (size_t i = 0; i < ds.size() && same; ++i) same = ds[i].first_chunk == (int64_t)i * per;
            *uniform = same ? (int)per : 0;
            return ds;
        };
        e.chain_chunks = e.direct_chain_chunks = 0;
        e.host.chain_segs = chain_segments(P.chain_segs, &e.chain_chunks, &e.chain_seg_chunks, &e.chain_tree, &e.chain_whole, &e.chain_alike);
        e.host.direct_chain_segs = chain_segments(P.direct_chain_segs, &e.direct_chain_chunks, &e.direct_chain_seg_chunks, &e.direct_chain_tree, &e.direct_chain_whole, &e.direct_chain_alike);
        e.host.chain_srcs.assign(P.chain_srcs.begin(), P.chain_srcs.end());
        if (e.host.chain_srcs.size() % 2) e.host.chain_srcs.push_back(0);
    }
    if (!P.gather.empty()) {
        std::vector<DevGatherCopy> gc(P.gather.size());
        int64_t tiles = 0;
        for (size_t i = 0; i < gc.size(); ++i) {
            const Program::GatherCopy& g = P.gather[i];
            gc[i].src_rank = g.src_rank; gc[i].dst_rank = g.dst_rank;
            gc[i].src_off = g.src_off * es; gc[i].dst_off = g.dst_off * es; gc[i].bytes = g.elems * es;
            gc[i].first_tile = tiles;
            tiles += (gc[i].bytes + 4095) / 4096;
        }
        e.gather_tiles = tiles;
        // all copies the same number of tiles (an alltoall's equal chunks)?
        const int64_t per = gc.size() > 1 ? gc[1].first_tile : tiles;
        e.gather_copy_tiles = 0;
        bool same = per > 0 && tiles == per * (int64_t)gc.size() && tiles <= INT32_MAX;
        for (size_t i = 0; i < gc.size() && same; ++i) same = gc[i].first_tile == (int64_t)i * per;
        if (same) e.gather_copy_tiles = (int)per;
        e.host.gather = std::move(gc);
    }
    // stepwise plan
    {
        std::vector<DevStepOp> so(P.ops.size());
        std::vector<int32_t> item_op((size_t)P.num_items);
        for (size_t k = 0; k < P.ops.size(); ++k) {
            const LinkedOp& L = P.ops[k];
            DevStepOp& d = so[k];
            d.off0 = L.off0; d.off1 = L.off1; d.off2 = L.off2; d.size = L.size;
            d.who = (uint32_t)L.rank | (uint32_t)L.peer << 8 | (uint32_t)(L.is_reduce ? 1 : 0) << 16 | (uint32_t)L.redop << 24;
            d.first_item = P.step_ops[k].first_item; d.ntiles = P.step_ops[k].ntiles;
            d.dep_start = P.step_ops[k].dep_start; d.ndeps = P.step_ops[k].ndeps;
            d.lead = P.step_ops[k].lead; d.pad_[0] = d.pad_[1] = 0;
            if (d.ndeps > 256) throw Error{PCCL_ERR_UNSUPPORTED, "a data op with more than 256 direct predecessors"};
            for (int t = 0; t < d.ntiles; ++t) item_op[(size_t)d.first_item + t] = (int32_t)k;
        }
        e.level_item_begin.clear();
        for (size_t k = 0; k < P.ops.size(); ++k)
            if (k == 0 || P.ops[k].level != P.ops[k - 1].level) e.level_item_begin.push_back(P.step_ops[k].first_item);
        e.level_item_begin.push_back((int)P.num_items);
        e.host.step_ops = std::move(so);
        e.host.item_op = std::move(item_op);
        e.host.step_deps_padded = P.step_deps;
        if (e.host.step_deps_padded.size() % 2) e.host.step_deps_padded.push_back(0);
    }
    static std::atomic<uint64_t> link_counter{0};
    e.generation = ++link_counter;
    e.host_linked = true;
    warn_about(P, "operation linked over " + std::to_string(ctx->R) + " virtual ranks", ctx->check_races);
    if (log_threshold() <= LOG_INFO)   // the reference's "Fused step executor enabled" line (engine_c.cc:357)
        log_line(LOG_INFO, "linked " + std::to_string(ctx->R) + " rank graphs: " + std::to_string(P.ops.size()) + " data ops on " +
                               std::to_string(P.num_levels) + " levels, " + std::to_string(P.num_items) + " work items of " +
                               std::to_string(P.tile_elems * es) + " bytes; " +
                               (P.position_aligned ? "position aligned, " + std::to_string(P.segs.size()) + " column segments, " +
                                                         (e.slot_threads > 0 ? "slot runner with " + std::to_string(e.slot_threads) + " threads"
                                                                             : std::string("register runner"))
                                                   : std::string("not position aligned: level / persistent runner")) +
                               (P.gather.empty() ? "" : "; alltoall gather plan of " + std::to_string(P.gather.size()) + " copies"));
}

// Device half: upload the tables (allocations and copies, hence never on a capturing stream).
void link_entry(pccl_hip_ctx* ctx, OpEntry& e, hipStream_t stream = nullptr, bool check_stream = false) {
    if (e.linked) return;
    if (check_stream) refuse_setup_under_capture(stream, "upload the operation's plan tables");
    link_host(ctx, e);
    const Program& P = e.prog;
    const OpEntry::HostTables& h = e.host;
    e.segs.upload(h.segs.data(), h.segs.size() * sizeof(DevColSegment));
    e.direct_segs.upload(h.direct_segs.data(), h.direct_segs.size() * sizeof(DevColSegment));
    if (P.position_aligned) {
        e.instrs.upload(P.col_instrs.data(), P.col_instrs.size() * sizeof(ColInstr));
        e.pre.upload(P.col_pre.data(), P.col_pre.size() * sizeof(uint64_t));
    }
    e.gather.upload(h.gather.data(), h.gather.size() * sizeof(DevGatherCopy));
    e.chain_segs.upload(h.chain_segs.data(), h.chain_segs.size() * sizeof(DevChainSegment));
    e.direct_chain_segs.upload(h.direct_chain_segs.data(), h.direct_chain_segs.size() * sizeof(DevChainSegment));
    e.chain_srcs.upload(h.chain_srcs.data(), h.chain_srcs.size() * sizeof(int32_t));
    if (!h.chain_segs.empty() || !h.direct_chain_segs.empty()) {
        const PhaseSync zero{};
        e.phase_sync.upload(&zero, sizeof(zero));
    }
    e.step_ops.upload(h.step_ops.data(), h.step_ops.size() * sizeof(DevStepOp));
    e.step_deps.upload(P.step_deps.data(), P.step_deps.size() * sizeof(int32_t));
    e.item_op.upload(h.item_op.data(), h.item_op.size() * sizeof(int32_t));
    std::vector<char> zeros(sizeof(StepState) + sizeof(int32_t) * ((size_t)P.num_items + P.ops.size() + 1), 0);
    e.state.upload(zeros.data(), zeros.size());
    e.epoch = 0;
    HIP_TRY(hipEventCreate(&e.ev0));
    HIP_TRY(hipEventCreate(&e.ev1));
    e.linked = true;
}

// How the slot runner stores a program's final broadcast.  A plan that writes far more than it reads
// (an allgather: one chunk in, R out) gains from whole tiles of a rank going out from one wave
// (8 ranks x 512 MB fp16 allgather 0.82 -> 0.79 ms); plans that read as much as they write are the
// same either way, and with fewer than four waves in a workgroup the ranks queue up behind each
// other (32-rank tree 1.12 -> 1.28 ms).
int store_waves(const pccl_hip_ctx* ctx, const OpEntry& e, int64_t load_bytes, int64_t store_bytes) {
    if (ctx->slot_store_waves >= 0) return ctx->slot_store_waves;
    return e.slot_threads >= 256 && store_bytes >= 4 * load_bytes ? 1 : 0;
}

OpEntry& find_entry(pccl_hip_ctx* ctx, const char* name) {
    auto it = ctx->ops.find(name ? name : "");
    if (it == ctx->ops.end()) throw Error{PCCL_ERR_NOT_FOUND, std::string("Unknown operation: ") + (name ? name : "(null)")};
    return it->second;
}

// The level runner: one launch per dependency level, or - option level_graph - the launches of an
// execution replayed as one HIP graph.  The graph holds only kernel nodes (no memset nodes), is
// captured on a private stream and is bound to one set of rank pointers (kernel arguments are
// frozen at capture time); a handful are kept per operation, the least recently used is dropped.
int launch_levels(pccl_hip_ctx* ctx, OpEntry& e, const StepwiseLaunch& L, const RankPtrs& ptrs, char* const* rank_bufs,
                  hipStream_t stream) {
    const size_t nlevels = e.level_item_begin.size() - 1;
    auto launch_all = [&](hipStream_t s) {
        int rc = 0;
        for (size_t l = 0; l < nlevels && rc == 0; ++l)
            rc = launch_level(L, e.level_item_begin[l], e.level_item_begin[l + 1], ptrs, s);
        return rc;
    };
    if (!ctx->level_graph || e.graph_failed || nlevels < 2 || is_capturing(stream)) return launch_all(stream);

    std::vector<char*> key(rank_bufs, rank_bufs + ctx->R);
    OpEntry::LevelGraph* hit = nullptr;
    for (auto& g : e.level_graphs) if (g.key == key) hit = &g;
    if (!hit) {
        if (!ctx->capture_stream) HIP_TRY(hipStreamCreateWithFlags(&ctx->capture_stream, hipStreamNonBlocking));
        OpEntry::LevelGraph g;
        g.key = key;
        hipError_t st = hipStreamBeginCapture(ctx->capture_stream, hipStreamCaptureModeThreadLocal);
        if (st == hipSuccess) {
            const int lrc = launch_all(ctx->capture_stream);
            st = hipStreamEndCapture(ctx->capture_stream, &g.graph);
            if (st == hipSuccess && lrc != 0) st = (hipError_t)lrc;
        }
        if (st == hipSuccess) st = hipGraphInstantiate(&g.exec, g.graph, nullptr, nullptr, 0);
        if (st != hipSuccess) {   // capture does not work here: launch level by level from now on
            if (g.exec) (void)hipGraphExecDestroy(g.exec);
            if (g.graph) (void)hipGraphDestroy(g.graph);
            (void)hipGetLastError();
            e.graph_failed = true;
            return launch_all(stream);
        }
        if (e.level_graphs.size() >= 4) {
            size_t old = 0;
            for (size_t i = 1; i < e.level_graphs.size(); ++i) if (e.level_graphs[i].used < e.level_graphs[old].used) old = i;
            (void)hipGraphExecDestroy(e.level_graphs[old].exec);
            (void)hipGraphDestroy(e.level_graphs[old].graph);
            e.level_graphs.erase(e.level_graphs.begin() + old);
        }
        e.level_graphs.push_back(g);
        hit = &e.level_graphs.back();
    }
    hit->used = ++e.graph_clock;
    return (int)hipGraphLaunch(hit->exec, stream);
}

// Whether a column-mode execution goes to the phased runner, and its launch.  `direct`: the staged
// call's plan on the caller's tensors.  The phased runner pays from about one 128 KiB chunk of every
// rank per CU on (8-rank bf16 ring allreduce, in place: 16 MiB per rank 54 us on either runner, 32 MiB
// 88 against 97 us, 128 MiB 0.344 against 0.359 ms); smaller tensors stay with the slot runner, whose
// many small workgroups start and end faster (4 MiB per rank: 17 against 44 us).
// Whether the plan can run with the chunks of 128 neighbouring workgroups interleaved slab by slab
// (phased_kernel_linear), and in groups of how many: chains on up to 8 ranks, every segment a whole
// multiple of 128 chunks and a grid that 128 divides; 0 if it cannot.
constexpr int kLinearGroup = 128;
int linear_group(const pccl_hip_ctx* ctx, const OpEntry& e, bool direct, int* group_segs = nullptr);
bool linear_fits(const pccl_hip_ctx* ctx, const OpEntry& e, bool direct) { return linear_group(ctx, e, direct) > 0; }
int linear_group(const pccl_hip_ctx* ctx, const OpEntry& e, bool direct, int* group_segs) {
    if (group_segs) *group_segs = 1;
    const int64_t chunks = direct ? e.direct_chain_chunks : e.chain_chunks;
    const int seg_chunks = direct ? e.direct_chain_seg_chunks : e.chain_seg_chunks;
    const int tree_shape = direct ? e.direct_chain_tree : e.chain_tree;
    const bool whole = direct ? e.direct_chain_whole : e.chain_whole;
    int64_t grid = ctx->num_blocks > 0 ? ctx->num_blocks : device_cu_count(ctx->device);
    if (grid > chunks) grid = chunks;
    if (tree_shape || ctx->R > 8 || !whole || seg_chunks <= 0 || grid <= 0) return 0;
    if (seg_chunks % kLinearGroup == 0 && grid % kLinearGroup == 0) return kLinearGroup;
    // shorter segments: a group spans two of them - four for plans that mostly write - if they are alike
    // (the rows of a group then belong to different segments: phased_kernel_linear_rows).  8-rank bf16
    // ring in place on 4 channels against the two-sweep shape, fraction of peak: segments of 64 chunks
    // (256 MiB per rank) 0.794-0.796 -> 0.816-0.819; of 32 chunks 0.784 / 0.816 -> 0.7855 / 0.7925; of 16
    // chunks 0.777-0.784 -> 0.764.  fp16 allgather against the slot runner: 8 x 64 MB 0.733 -> 0.758-0.767,
    // 8 x 32 MB 0.696-0.698 -> 0.711-0.713.
    const bool alike = direct ? e.direct_chain_alike : e.chain_alike;
    const int64_t loads = direct ? e.prog.direct_slot_load_bytes : e.prog.slot_load_bytes;
    const int64_t stores = direct ? e.prog.direct_slot_store_bytes : e.prog.slot_store_bytes;
    const bool mostly_writes = 2 * loads < stores;
    if (alike && grid % kLinearGroup == 0 && chunks % kLinearGroup == 0 && (seg_chunks == 64 || (seg_chunks == 32 && mostly_writes))) {
        if (group_segs) *group_segs = kLinearGroup / seg_chunks;
        return kLinearGroup;
    }
    // groups of 64 where that is not possible (segments of 64 chunks that are not alike): worth it for
    // plans that mostly write only (8 x 64 MB fp16 allgather 0.727-0.729 -> 0.738-0.741 of peak)
    if (mostly_writes && seg_chunks % 64 == 0 && grid % 64 == 0) return 64;
    return 0;
}

bool wants_phased(const pccl_hip_ctx* ctx, const OpEntry& e, bool direct) {
    const int64_t chunks = direct ? e.direct_chain_chunks : e.chain_chunks;
    const DevBuf& segs = direct ? e.direct_chain_segs : e.chain_segs;
    if (ctx->phased == 0 || chunks <= 0 || !segs.p || !e.phase_sync.p) return false;
    if (ctx->phased == 1) return true;
    // a plan that mostly writes (an allgather: one chunk in, R out) has no read phase to speak of and
    // is faster with the slot runner's wave-dealt stores (8 x 512 MB fp16: 0.80 against 0.83-0.86 ms) -
    // unless its chunks can be interleaved, which is what its writes gain from (8 x 128 / 256 / 512 MB:
    // 0.773 / 0.77 / 0.759 of peak against 0.75 / 0.735-0.74 / 0.76 on the slot runner)
    const int64_t loads = direct ? e.prog.direct_slot_load_bytes : e.prog.slot_load_bytes;
    const int64_t stores = direct ? e.prog.direct_slot_store_bytes : e.prog.slot_store_bytes;
    if (2 * loads < stores) return ctx->phased_linear != 0 && ctx->phased_shape < 0 && ctx->phased_sweeps < 0 && linear_fits(ctx, e, direct);
    // it pays from one chunk per two CUs on (8-rank bf16 ring in place: 16 MiB per rank, 128 chunks,
    // 0.613 -> 0.637 of peak; 32 MiB 0.679 -> 0.748; 8 MiB 0.563 -> 0.368.  8-rank fp16 reduce_scatter:
    // 16 MB per rank 32.6 -> 29.3 us, 8 MB 18.6 -> 25.8).  Quarter chunks for the sizes below were
    // measured (512 threads x 4 vectors) and are no better than the slot runner there.
    return 2 * chunks >= (int64_t)device_cu_count(ctx->device);
}

// The launch record of the phased runner for this operation's chain plan: which of its shapes, with
// what grouping and whether with meetings (the one place that decides it).
PhasedLaunch phased_launch_for(pccl_hip_ctx* ctx, OpEntry& e, bool direct) {
    const Program& P = e.prog;
    PhasedLaunch L{};
    L.segs = (const DevChainSegment*)(direct ? e.direct_chain_segs.p : e.chain_segs.p);
    L.num_segs = (int)(direct ? P.direct_chain_segs.size() : P.chain_segs.size());
    L.srcs = (const int32_t*)e.chain_srcs.p;
    L.total_chunks = direct ? e.direct_chain_chunks : e.chain_chunks;
    L.seg_chunks = direct ? e.direct_chain_seg_chunks : e.chain_seg_chunks;
    L.dtype = P.dtype;
    // 8 ranks and fewer: two waves per SIMD with 16 vectors each; more ranks: one wave per SIMD that
    // streams 32 KiB of every rank in a row (measured with bare kernels: 8 ranks 80 % against 78 % of
    // peak, 32 ranks 81 % against 83 %)
    const int tree_shape = direct ? e.direct_chain_tree : e.chain_tree;
    L.shape = tree_shape ? tree_shape : ctx->phased_shape >= 0 ? ctx->phased_shape : (ctx->R <= 8 ? 0 : 1);
    // 256 x 32 chains read as slabs and write with each wave on 32 KiB in a row, the sums changing hands
    // through LDS between the phases (32 ranks x 96 MiB: int32 SUM 0.822 -> 0.842 of peak, f32 MAX
    // 0.820 -> 0.840; 16-rank bf16 ring 0.335 -> 0.327 ms); trees gain nothing from it and keep their shape
    if (ctx->phased_exchange != 0 && L.shape == 1) L.shape = 3;
    L.num_blocks = ctx->num_blocks;
    // a plan that mostly reads (a reduce_scatter: R chunks in, one out) has write phases too short to be
    // worth a meeting per sweep (8 x 64 MB fp16: 89 us without, 94 us with).  It reads two sweeps in one
    // fetch stream and then writes both (shape 4: bare kernels of that traffic, 8 x 512 MiB in, 8 x
    // 64 MiB out, 0.788 of peak without meetings, 0.804 with one write phase per sweep, 0.865 per two
    // sweeps, 0.868 per three), from two sweeps on; below, it runs without meetings
    const int64_t loads = direct ? P.direct_slot_load_bytes : P.slot_load_bytes;
    const int64_t stores = direct ? P.direct_slot_store_bytes : P.slot_store_bytes;
    const bool mostly_reads = loads >= 4 * stores;
    // (8-rank fp16 reduce_scatter, one sweep per write phase without meetings -> two with: 512 / 256 /
    // 128 / 64 MB per rank 0.805 -> 0.852, 0.831 -> 0.846, 0.834 -> 0.844, 0.832 -> 0.846 of peak; 32 / 16 MB,
    // one sweep and half a one, 0.815 -> 0.764 / 0.619 -> 0.547).  The 512 x 16 shape of the other
    // chains (up to 8 ranks) gains from it as well, from two sweeps on: fewer, longer phases (8-rank ring
    // in place, 512 MiB per rank: bf16 0.778 -> 0.790, f16 0.770 -> 0.787, f32 0.782 -> 0.792, int32
    // 0.788 -> 0.795 on one box; bf16 64 / 128 / 256 MiB 0.771 -> 0.785, 0.784 -> 0.784, 0.791 -> 0.799)
    const int64_t cus = device_cu_count(ctx->device);
    const bool pays = L.total_chunks >= 2 * cus && (mostly_reads || L.shape == 0);
    const bool two_sweeps = !tree_shape && (ctx->phased_sweeps == 2 || (ctx->phased_sweeps < 0 && ctx->phased_shape < 0 && pays));
    if (two_sweeps) L.shape = 4;
    // Chains on up to 8 ranks whose segments are whole multiples of 128 chunks (16 MiB of every rank): the
    // chunks of 128 neighbouring workgroups interleaved slab by slab, so that the chip sweeps each rank
    // buffer as one linear stream (shape 5; headline 0.797-0.800 -> 0.825-0.828 of peak in alternating runs
    // on one box).  Plans that mostly read keep the two-sweep shape: their gain is on the read side.
    L.group = 0;
    {
        const bool wanted = ctx->phased_linear == 1 || (ctx->phased_linear < 0 && ctx->phased_shape < 0 && ctx->phased_sweeps < 0 && !mostly_reads);
        if (wanted && linear_fits(ctx, e, direct)) { int gs = 1; L.shape = 5; L.group = linear_group(ctx, e, direct, &gs); L.group_segs = gs; }
    }
    L.barriers = ctx->phased_barriers && (two_sweeps || L.shape == 5 || !mostly_reads) ? 1 : 0;
    L.sync = (PhaseSync*)e.phase_sync.p;
    L.timeout_ticks = (uint64_t)ctx->phased_timeout_us * 100ull;
    return L;
}

int launch_phased_plan(pccl_hip_ctx* ctx, OpEntry& e, bool direct, const RankPtrs& ptrs, hipStream_t stream) {
    return launch_phased(phased_launch_for(ctx, e, direct), ptrs, stream);
}

// Enqueue the program on `stream` over the rank buffers `rank_bufs` (R pointers).
void run_program(pccl_hip_ctx* ctx, OpEntry& e, char* const* rank_bufs, size_t buf_bytes, hipStream_t stream) {
    const Program& P = e.prog;
    const int es = elem_size(P.dtype);
    if ((size_t)P.buffer_elems * es > buf_bytes)
        throw Error{PCCL_ERR_INVALID, "rank buffers of " + std::to_string(buf_bytes) + " bytes are smaller than the " + std::to_string((size_t)P.buffer_elems * es) + " bytes the graph addresses"};
    if (P.ops.empty()) return;
    RankPtrs ptrs;
    std::memset(&ptrs, 0, sizeof(ptrs));
    bool aligned16 = true;
    for (int r = 0; r < ctx->R; ++r) {
        if (!rank_bufs[r]) throw Error{PCCL_ERR_INVALID, "null rank buffer " + std::to_string(r)};
        if ((uintptr_t)rank_bufs[r] % es) throw Error{PCCL_ERR_INVALID, "rank buffer " + std::to_string(r) + " is not aligned to the element size"};
        if ((uintptr_t)rank_bufs[r] & 15) aligned16 = false;
        ptrs.p[r] = rank_bufs[r];
        ptrs.p[PCCL_HIP_MAX_VRANKS + r] = rank_bufs[r];
    }
    bool column = P.position_aligned && aligned16;
    if (ctx->mode == Mode::Stepwise || ctx->mode == Mode::Persistent) column = false;
    if (ctx->mode == Mode::Column && !column)
        throw Error{PCCL_ERR_UNSUPPORTED, P.position_aligned ? "column mode needs 16-byte aligned rank buffers" : "column mode needs every data op to read and write the same element positions"};
    if (ctx->timing) HIP_TRY(hipEventRecord(e.ev0, stream));
    int rc;
    TraceRange range(ctx->trace_ranges, column ? "fused_kernel" : "executor_kernel");
    if (column && wants_phased(ctx, e, false)) {
        rc = launch_phased_plan(ctx, e, false, ptrs, stream);
    } else if (column) {
        ColumnLaunch L{};
        L.segs = (const DevColSegment*)e.segs.p; L.num_segs = (int)P.segs.size();
        L.instrs = (const uint64_t*)e.instrs.p; L.pre = (const uint64_t*)e.pre.p;
        L.slot_threads = e.slot_threads; L.slot_vecs = e.slot_vecs; L.slot_lds_bytes = e.slot_lds_bytes; L.num_ranks = ctx->R; L.slot_direct = ctx->slot_direct;
        L.slot_store_waves = store_waves(ctx, e, P.slot_load_bytes, P.slot_store_bytes);
        L.total_tiles = e.total_tiles; L.seg_tiles = e.seg_tiles; L.dtype = P.dtype; L.vecs_per_thread = e.vecs_per_thread;
        L.num_blocks = ctx->num_blocks;
        rc = launch_column(L, ptrs, stream);
    } else {
        StepwiseLaunch L{};
        L.ops = (const DevStepOp*)e.step_ops.p; L.num_ops = (int)P.ops.size();
        L.deps = (const int32_t*)e.step_deps.p; L.item_op = (const int32_t*)e.item_op.p;
        L.num_items = (int)P.num_items; L.tile_elems = P.tile_elems; L.state = (StepState*)e.state.p;
        L.dtype = P.dtype; L.num_blocks = ctx->num_blocks;
        if (ctx->mode == Mode::Persistent) {
            // The launch number is a kernel argument, which every replay of a recorded launch would
            // repeat (finding all flags of the previous replay set): on a capturing stream the
            // number comes from a device-side counter that a one-thread kernel advances first.
            if (is_capturing(stream)) L.epoch = 0;
            else {
                if (e.epoch >= ctx->host_epoch_limit) {
                    // the launch numbers have run out: clear the flags and ready words (a fill kernel on the
                    // stream, behind every earlier launch) and count from 1 again
                    const int frc = launch_fill_zero((char*)e.state.p + sizeof(StepState), sizeof(int32_t) * ((size_t)P.num_items + P.ops.size() + 1), stream);
                    if (frc != 0) throw Error{PCCL_ERR_HIP, std::string("clearing the progress flags: ") + hipGetErrorString((hipError_t)frc)};
                    e.epoch = 0;
                }
                L.epoch = ++e.epoch;
            }
            L.graph_epoch_limit = ctx->graph_epoch_limit;
            L.timeout_ticks = (uint64_t)ctx->wait_timeout_ms * 100000ull;
            rc = launch_persistent(L, ptrs, stream);   // sizes the grid to what is resident at once
            e.ran_persistent = true;
        } else {
            rc = launch_levels(ctx, e, L, ptrs, rank_bufs, stream);
        }
    }
    if (rc != 0) throw Error{PCCL_ERR_HIP, std::string("kernel launch failed: ") + hipGetErrorString((hipError_t)rc)};
    if (ctx->timing) { HIP_TRY(hipEventRecord(e.ev1, stream)); e.timed = true; }
}

// Staged semantics without staging copies: first-touch loads read the caller's inputs, every store
// goes to the caller's outputs.  Returns false when the call does not qualify (the caller then
// stages through the engine's rank buffers).
bool run_direct(pccl_hip_ctx* ctx, OpEntry& e, const void* const* inputs, void* const* outputs,
                size_t in_bytes, size_t out_bytes, hipStream_t stream) {
    const Program& P = e.prog;
    if (!ctx->fuse_staging || ctx->mode == Mode::Stepwise || ctx->mode == Mode::Persistent) return false;
    if (!P.position_aligned || P.direct_segs.empty() || !e.direct_segs.p) return false;
    const size_t es = elem_size(P.dtype);
    // the tensors must be exactly the windows the plan was built for
    const size_t want_in = (size_t)(P.direct_in_end[0] - P.direct_in_start[0]) * es;
    const size_t want_out = (size_t)(P.direct_out_end[0] - P.direct_out_start[0]) * es;
    if (in_bytes != want_in || out_bytes < want_out) return false;
    const bool same_windows = P.direct_in_start == P.direct_out_start && P.direct_in_end == P.direct_out_end;
    RankPtrs ptrs;
    std::memset(&ptrs, 0, sizeof(ptrs));
    for (int r = 0; r < ctx->R; ++r) {
        uintptr_t in = (uintptr_t)inputs[r], out = (uintptr_t)outputs[r];
        // position p of rank r lives at base + p*es: shift the bases by the window starts
        uintptr_t in_base = in - (uintptr_t)P.direct_in_start[r] * es, out_base = out - (uintptr_t)P.direct_out_start[r] * es;
        if ((in_base | out_base) & 15) return false;
        bool aliased = in == out && same_windows;   // in place: every position read before it is written
        if (!aliased && in < out + want_out && out < in + in_bytes) return false;
        for (int q = 0; q < r; ++q) {  // an output must not alias another rank's tensors
            uintptr_t oq = (uintptr_t)outputs[q], iq = (uintptr_t)inputs[q];
            if ((out < oq + want_out && oq < out + want_out) || (out < iq + in_bytes && iq < out + want_out) ||
                (oq < in + in_bytes && in < oq + want_out)) return false;
        }
        ptrs.p[r] = (char*)out_base;
        ptrs.p[PCCL_HIP_MAX_VRANKS + r] = (char*)in_base;
    }
    if (ctx->timing) HIP_TRY(hipEventRecord(e.ev0, stream));
    if (wants_phased(ctx, e, true)) {
        TraceRange exe(ctx->trace_ranges, "execute"), range(ctx->trace_ranges, "fused_kernel");
        const int prc = launch_phased_plan(ctx, e, true, ptrs, stream);
        if (prc != 0) throw Error{PCCL_ERR_HIP, std::string("kernel launch failed: ") + hipGetErrorString((hipError_t)prc)};
        if (ctx->timing) { HIP_TRY(hipEventRecord(e.ev1, stream)); e.timed = true; }
        return true;
    }
    ColumnLaunch L{};
    L.segs = (const DevColSegment*)e.direct_segs.p; L.num_segs = (int)P.direct_segs.size();
    L.instrs = (const uint64_t*)e.instrs.p; L.pre = (const uint64_t*)e.pre.p;
    L.slot_threads = e.slot_threads; L.slot_vecs = e.slot_vecs; L.slot_lds_bytes = e.slot_lds_bytes; L.num_ranks = ctx->R; L.slot_direct = ctx->slot_direct;
    L.slot_store_waves = store_waves(ctx, e, P.direct_slot_load_bytes, P.direct_slot_store_bytes);
    L.total_tiles = e.direct_tiles; L.seg_tiles = e.direct_seg_tiles; L.dtype = P.dtype; L.vecs_per_thread = e.vecs_per_thread;
    L.num_blocks = ctx->num_blocks;
    TraceRange exe(ctx->trace_ranges, "execute"), range(ctx->trace_ranges, "fused_kernel");
    int rc = launch_column(L, ptrs, stream);
    if (rc != 0) throw Error{PCCL_ERR_HIP, std::string("kernel launch failed: ") + hipGetErrorString((hipError_t)rc)};
    if (ctx->timing) { HIP_TRY(hipEventRecord(e.ev1, stream)); e.timed = true; }
    return true;
}

// An alltoall as direct copies from the input tensors to the output tensors, when the program
// composes into such copies (the gather plan) and no output overlaps an input or another output.
bool run_gather(pccl_hip_ctx* ctx, OpEntry& e, const void* const* inputs, void* const* outputs,
                size_t in_bytes, size_t out_bytes, hipStream_t s) {
    const Program& P = e.prog;
    const int R = ctx->R;
    const size_t es = elem_size(P.dtype);
    if (P.collective_type != "alltoall" || !ctx->fuse_staging || !e.gather.p || ctx->mode != Mode::Auto ||
        in_bytes != (size_t)P.tensor_elems * es || out_bytes < in_bytes)
        return false;
    for (int r = 0; r < R; ++r)
        for (int q = 0; q < R; ++q) {
            const uintptr_t o = (uintptr_t)outputs[r], i = (uintptr_t)inputs[q];
            if (o < i + in_bytes && i < o + in_bytes) return false;
            if (q != r && o < (uintptr_t)outputs[q] + in_bytes && (uintptr_t)outputs[q] < o + in_bytes) return false;
        }
    RankPtrs src{}, dst{};
    for (int r = 0; r < R; ++r) { src.p[r] = (char*)inputs[r]; dst.p[r] = (char*)outputs[r]; }
    if (ctx->timing) HIP_TRY(hipEventRecord(e.ev0, s));
    TraceRange exe(ctx->trace_ranges, "execute"), range(ctx->trace_ranges, "fused_kernel");
    int rc = launch_gather((const DevGatherCopy*)e.gather.p, (int)P.gather.size(), e.gather_tiles, e.gather_copy_tiles, src, dst, s);
    if (rc) throw Error{PCCL_ERR_HIP, std::string("gather launch failed: ") + hipGetErrorString((hipError_t)rc)};
    if (ctx->timing) { HIP_TRY(hipEventRecord(e.ev1, s)); e.timed = true; }
    return true;
}

// The reference's staging (engine_c.cc:468-548): inputs into the rank buffers, the program, the
// results out of the rank buffers, laid out per collective type.
void run_staged(pccl_hip_ctx* ctx, OpEntry& e, const void* const* inputs, void* const* outputs,
                size_t in_bytes, size_t out_bytes, hipStream_t s) {
    const Program& P = e.prog;
    const int R = ctx->R;
    const size_t es = elem_size(P.dtype);
    const std::string& ct = P.collective_type;
    // the output must hold what the collective hands back; checked before anything is enqueued
    if (ct == "reduce_scatter" && out_bytes < in_bytes / R) throw Error{PCCL_ERR_INVALID, "reduce_scatter output is smaller than one chunk"};
    if (ct == "alltoall" && out_bytes < in_bytes / R * R) throw Error{PCCL_ERR_INVALID, "alltoall output is smaller than the input"};

    size_t need = (size_t)P.buffer_elems * es;
    if (ct == "allgather") need = std::max(need, in_bytes * R);
    else need = std::max(need, in_bytes);
    if (ct == "alltoall") need = std::max(need, 2 * in_bytes);
    else if (ct != "reduce_scatter") need = std::max(need, out_bytes);
    ensure_buffers(ctx, need, s);

    RankPtrs src{}, dst{}, bufp{};
    StageOffsets off{};
    for (int r = 0; r < R; ++r) {
        src.p[r] = (char*)inputs[r]; bufp.p[r] = ctx->bufs[r]; dst.p[r] = (char*)outputs[r];
        off.src[r] = 0;
        off.dst[r] = ct == "allgather" ? (int64_t)r * (int64_t)in_bytes : 0;
    }
    int rc;
    {
        TraceRange range(ctx->trace_ranges, "d2d_input_copy");
        rc = launch_stage(src, bufp, off, R, in_bytes, s);
    }
    if (rc) throw Error{PCCL_ERR_HIP, std::string("input staging: ") + hipGetErrorString((hipError_t)rc)};

    {
        TraceRange range(ctx->trace_ranges, "execute");
        run_program(ctx, e, ctx->bufs.data(), ctx->buf_bytes, s);
    }

    TraceRange range(ctx->trace_ranges, "d2d_output_copy");
    const size_t chunk = in_bytes / R;
    if (ct == "reduce_scatter") {           // chunk r of buffer r
        for (int r = 0; r < R; ++r) { off.src[r] = (int64_t)r * (int64_t)chunk; off.dst[r] = 0; }
        rc = launch_stage(bufp, dst, off, R, chunk, s);
    } else if (ct == "alltoall") {          // own chunk from the input region, the others from the scratch region
        rc = 0;
        for (int p = 0; p < R && rc == 0; ++p) {
            for (int r = 0; r < R; ++r) {
                off.src[r] = p == r ? (int64_t)r * (int64_t)chunk : (int64_t)in_bytes + (int64_t)p * (int64_t)chunk;
                off.dst[r] = (int64_t)p * (int64_t)chunk;
            }
            rc = launch_stage(bufp, dst, off, R, chunk, s);
        }
    } else {                                // allreduce and untyped graphs: the head of the buffer
        for (int r = 0; r < R; ++r) { off.src[r] = 0; off.dst[r] = 0; }
        rc = launch_stage(bufp, dst, off, R, out_bytes, s);
    }
    if (rc) throw Error{PCCL_ERR_HIP, std::string("output staging: ") + hipGetErrorString((hipError_t)rc)};
}

// After the stream has drained: did a bounded wait of the persistent runner expire?
void check_stall(OpEntry& e, const std::string& name) {
    if (!e.ran_persistent || !e.state.p) return;
    e.ran_persistent = false;
    StepState st;
    HIP_TRY(hipMemcpy(&st, e.state.p, sizeof(st), hipMemcpyDeviceToHost));
    if (st.error_op == 0) return;
    std::vector<char> zeros(e.state.bytes, 0);
    HIP_TRY(hipMemcpy(e.state.p, zeros.data(), zeros.size(), hipMemcpyHostToDevice));
    e.epoch = 0;
    const int n_ops = (int)e.prog.ops.size();
    if (st.error_op > n_ops || st.error_dep < 1 || st.error_dep > n_ops)
        throw Error{PCCL_ERR_HIP, "operation '" + name + "': the persistent runner gave up waiting (its progress block names ops " +
                                      std::to_string(st.error_op - 1) + " and " + std::to_string(st.error_dep - 1) + ", which the program does not have)"};
    const LinkedOp& a = e.prog.ops[st.error_op - 1];
    const LinkedOp& b = e.prog.ops[st.error_dep - 1];
    throw Error{PCCL_ERR_HIP, "operation '" + name + "': the persistent runner gave up waiting: data op " + std::to_string(st.error_op - 1) +
                                  " (rank " + std::to_string(a.rank) + ", level " + std::to_string(a.level) + ") never saw its predecessor " +
                                  std::to_string(st.error_dep - 1) + " (rank " + std::to_string(b.rank) + ", level " + std::to_string(b.level) +
                                  ") complete; rank buffers are partially updated"};
}

// ---- execution in the static workspace (no allocation anywhere in the call) -------------------
//
// What the persistent runner needs on the device besides the rank buffers - its progress block (error
// words, one flag per work item, one ready word per op) and its tables (ops, dependency lists,
// item -> op map) - laid out in the GPU's static workspace.  One such workspace exists per GPU and
// every call on that GPU uses it, whichever context or operation it comes from: the host remembers
// whose tables it holds and rewrites them when another operation takes it over.
struct StaticWorkspace {
    std::mutex mu;
    char* ptr = nullptr;          // device address on this GPU (asked for at pccl_hip_create, with the device current)
    size_t bytes = 0;
    uint64_t owner = 0;           // OpEntry::generation whose tables the workspace holds (0: none)
    int32_t epoch = 0;            // launches since the flags were last cleared
};

StaticWorkspace& static_ws(int device) {
    static StaticWorkspace ws[16];
    return ws[device >= 0 && device < 16 ? device : 0];
}

// What StepState::owner holds while the workspace carries the tables of `e`: never 0.
uint32_t static_tag(const OpEntry& e) { return (uint32_t)(e.generation & 0x7FFFFFFFu) | 0x80000000u; }

struct StaticLayout { size_t state, flags, ready, ops, deps, item_op, total; };

StaticLayout static_layout(const Program& P) {
    auto up = [](size_t x) { return (x + 255) & ~(size_t)255; };
    StaticLayout l{};
    l.state = 0;
    l.flags = sizeof(StepState);                                   // flags and ready words follow the block directly,
    l.ready = l.flags + sizeof(int32_t) * (size_t)P.num_items;      // as the kernel expects
    l.ops = up(l.ready + sizeof(int32_t) * (P.ops.size() + 1));
    l.deps = up(l.ops + sizeof(DevStepOp) * P.ops.size());
    l.item_op = up(l.deps + sizeof(int32_t) * (P.step_deps.size() + 2));
    l.total = up(l.item_op + sizeof(int32_t) * (size_t)P.num_items);
    return l;
}

// A recorded launch that was replayed after the workspace had gone to another operation has left
// its tag behind (it executed nothing and touched no buffer).  Whoever looks at the block next
// notes it: a WARN line that names the operation, the word is cleared, and the operation whose
// launch it was - if it belongs to this context - hears of it as an error at its own next
// pccl_hip_sync.  The call that happens to find the word is not failed: it executed normally.
void note_stale_launch(pccl_hip_ctx* ctx, StaticWorkspace& ws, const StepState& st) {
    if (st.stale_owner == 0) return;
    std::string who = "an operation of another context";
    for (auto& kv : ctx->ops)
        if (kv.second.generation != 0 && static_tag(kv.second) == st.stale_owner) {
            who = "operation '" + kv.first + "'";
            kv.second.stale_replay = true;
        }
    log_line(LOG_WARN, "a recorded launch of pccl_hip_execute_inplace_static (" + who + ") was replayed after the static workspace had been "
                       "taken over by another operation; that replay executed nothing and left its rank buffers as they were");
    const uint32_t zero = 0;
    HIP_TRY(hipMemcpy(ws.ptr + offsetof(StepState, stale_owner), &zero, sizeof(zero), hipMemcpyHostToDevice));
}

// The progress block of the static workspace after the stream has drained: a stall of THIS launch is
// an error (checked first, so that a stale replay seen in the same look never hides it); a stale
// replay is noted as above.
void read_static_block(pccl_hip_ctx* ctx, StaticWorkspace& ws, const std::string& name) {
    StepState st;
    HIP_TRY(hipMemcpy(&st, ws.ptr, sizeof(st), hipMemcpyDeviceToHost));
    const bool stalled = st.error_op != 0;
    if (stalled) ws.owner = 0;                         // the next call clears and rewrites everything
    note_stale_launch(ctx, ws, st);
    if (stalled)
        throw Error{PCCL_ERR_HIP, "operation '" + name + "': the persistent runner gave up waiting in the static workspace (data op " +
                                      std::to_string(st.error_op - 1) + " never saw its predecessor " + std::to_string(st.error_dep - 1) +
                                      " complete); rank buffers are partially updated"};
}

void check_stall_static(pccl_hip_ctx* ctx, OpEntry& e, const std::string& name) {
    if (e.ran_static) {
        e.ran_static = false;
        StaticWorkspace& ws = static_ws(ctx->device);
        std::lock_guard<std::mutex> lock(ws.mu);
        // (when another operation has taken the workspace over since, its own look covers the block)
        if (ws.ptr && ws.owner == e.generation) read_static_block(ctx, ws, name);
    }
    if (e.stale_replay) {
        e.stale_replay = false;
        throw Error{PCCL_ERR_INVALID, "a recorded launch of operation '" + name + "' (pccl_hip_execute_inplace_static) was replayed after the static "
                                      "workspace had been taken over by another operation: that replay executed nothing and left its rank buffers "
                                      "unchanged.  Execute the operation once through that entry point and the recorded launch works again"};
    }
}

int register_graph(pccl_hip_ctx* ctx, const char* name, int vrank, RankGraph&& g) {
    if (!ctx || !name) return fail(PCCL_ERR_INVALID, "null argument");
    if (vrank < 0 || vrank >= ctx->R) return fail(PCCL_ERR_INVALID, "virtual rank " + std::to_string(vrank) + " outside 0.." + std::to_string(ctx->R - 1));
    std::lock_guard<std::mutex> lock(ctx->mu);
    HIP_TRY(hipSetDevice(ctx->device));
    OpEntry& e = ctx->ops[name];
    if (e.graphs.empty()) e.graphs.resize(ctx->R);
    if (e.linked) HIP_TRY(hipDeviceSynchronize());
    if (e.linked || e.host_linked) e.release();  // re-registration replaces the op
    e.uses_scanned = false;
    e.graphs[vrank] = std::make_unique<RankGraph>(std::move(g));
    if (log_threshold() <= LOG_INFO)   // reference engine_c.cc:168,199
        log_line(LOG_INFO, std::string("operation '") + name + "' registered for virtual rank " + std::to_string(vrank) + ": " +
                               std::to_string(e.graphs[vrank]->ops.size()) + " ops");
    return 0;
}

}  // namespace

extern "C" {

int pccl_hip_create(pccl_hip_ctx** out, int device, int num_vranks) {
    return guarded([&] {
        if (!out) return fail(PCCL_ERR_INVALID, "null argument");
        if (num_vranks < 1 || num_vranks > PCCL_HIP_MAX_VRANKS)
            return fail(PCCL_ERR_INVALID, "num_vranks must be 1.." + std::to_string(PCCL_HIP_MAX_VRANKS));
        int count = 0;
        if (hipGetDeviceCount(&count) != hipSuccess || count <= 0)
            return fail(PCCL_ERR_HIP, "no HIP device is visible: the executor has no CPU fallback");
        if (device < 0 || device >= count) return fail(PCCL_ERR_INVALID, "device index out of range");
        HIP_TRY(hipSetDevice(device));
        auto ctx = std::make_unique<pccl_hip_ctx>();
        ctx->device = device;
        ctx->R = num_vranks;
        ctx->bufs.assign(num_vranks, nullptr);
        {   // the static workspace of this GPU: its address is asked for here, once per device, with the device current
            StaticWorkspace& ws = static_ws(device);
            std::lock_guard<std::mutex> lock(ws.mu);
            if (!ws.ptr) {
                void* p = nullptr;
                size_t n = 0;
                const int rc = static_workspace(device, &p, &n);
                if (rc != 0) return fail(PCCL_ERR_HIP, std::string("static workspace: ") + hipGetErrorString((hipError_t)rc));
                ws.ptr = (char*)p; ws.bytes = n;
            }
        }
        if (const char* nb = std::getenv("PCCL_NUM_BLOCKS")) ctx->num_blocks = std::atoi(nb);
        if (std::getenv("PCCL_DISABLE_FUSED")) ctx->mode = Mode::Stepwise;
        if (const char* tr = std::getenv("PCCL_TRACE_RANGES")) ctx->trace_ranges = std::atoi(tr) != 0;
        if (const char* ph = std::getenv("PCCL_PHASED")) { const int x = std::atoi(ph); if (x >= -1 && x <= 1) ctx->phased = x; }
        if (log_threshold() <= LOG_INFO)   // reference engine_c.cc:84,163
            log_line(LOG_INFO, "engine context on device " + std::to_string(device) + " with " + std::to_string(num_vranks) + " virtual ranks");
        *out = ctx.release();
        return 0;
    });
}

int pccl_hip_destroy(pccl_hip_ctx* ctx) {
    if (!ctx) return 0;
    (void)hipSetDevice(ctx->device);
    (void)hipDeviceSynchronize();
    for (auto& kv : ctx->ops) kv.second.release();
    for (char* b : ctx->bufs) if (b) (void)hipFree(b);
    if (ctx->capture_stream) (void)hipStreamDestroy(ctx->capture_stream);
    delete ctx;
    return 0;
}

int pccl_hip_register_file(pccl_hip_ctx* ctx, const char* name, int vrank, const char* path) {
    return guarded([&] {
        if (!path) return fail(PCCL_ERR_INVALID, "null path");
        return register_graph(ctx, name, vrank, load_graph_file(path));
    });
}

int pccl_hip_register_json(pccl_hip_ctx* ctx, const char* name, int vrank, const char* text, size_t len) {
    return guarded([&] {
        if (!text) return fail(PCCL_ERR_INVALID, "null text");
        return register_graph(ctx, name, vrank, load_graph_json(text, len));
    });
}

int pccl_hip_register_triggers(pccl_hip_ctx* ctx, const char* name, int vrank, const pccl_trigger* triggers,
                               const pccl_primitive_meta* meta, int n, const char* collective_type) {
    return guarded([&] { return register_graph(ctx, name, vrank, graph_from_triggers(triggers, meta, n, collective_type)); });
}

// An option value that has to be a whole number: "on", "True" or "4x" are refused, not read as 0 or 4.
static long long whole_number(const std::string& key, const char* value) {
    errno = 0;
    char* end = nullptr;
    const long long x = std::strtoll(value, &end, 10);
    if (end == value || *end != '\0' || errno != 0)
        throw Error{PCCL_ERR_INVALID, "option '" + key + "' takes a whole number, got '" + value + "'"};
    return x;
}
static int int_value(const std::string& key, const char* value) {
    const long long x = whole_number(key, value);
    if (x < INT32_MIN || x > INT32_MAX) throw Error{PCCL_ERR_INVALID, "option '" + key + "': " + value + " is out of range"};
    return (int)x;
}

int pccl_hip_set_option(pccl_hip_ctx* ctx, const char* key, const char* value) {
    return guarded([&] {
        if (!ctx || !key || !value) return fail(PCCL_ERR_INVALID, "null argument");
        std::lock_guard<std::mutex> lock(ctx->mu);
        std::string k = key, v = value;
        bool relink = false;
        if (k == "mode") {
            if (v == "auto") ctx->mode = Mode::Auto;
            else if (v == "column") ctx->mode = Mode::Column;
            else if (v == "stepwise") ctx->mode = Mode::Stepwise;
            else if (v == "persistent") ctx->mode = Mode::Persistent;
            else return fail(PCCL_ERR_INVALID, "mode must be auto, column, stepwise or persistent");
        } else if (k == "num_blocks") ctx->num_blocks = int_value(k, value);
        else if (k == "timing") ctx->timing = int_value(k, value) != 0;
        else if (k == "trace_ranges") {
            ctx->trace_ranges = int_value(k, value) != 0;
            if (ctx->trace_ranges && !marker_api().push) { ctx->trace_ranges = false; return fail(PCCL_ERR_UNSUPPORTED, "trace_ranges: no roctx marker library could be loaded"); }
        }
        else if (k == "fuse_staging") ctx->fuse_staging = int_value(k, value) != 0;
        else if (k == "wait_timeout_ms") { ctx->wait_timeout_ms = int_value(k, value); if (ctx->wait_timeout_ms < 0) ctx->wait_timeout_ms = 0; }   // 0: give up on the first predecessor that is not ready
        else if (k == "test_host_epoch_limit" || k == "test_graph_epoch_limit") {
            // for tests: bring the point where the persistent runner's launch numbers wrap within reach
            const long long x = whole_number(k, value);
            if (k == "test_host_epoch_limit") {
                if (x < 2 || x > kHostEpochLimit) return fail(PCCL_ERR_INVALID, "test_host_epoch_limit must be 2 .. " + std::to_string(kHostEpochLimit));
                ctx->host_epoch_limit = (int32_t)x;
            } else {
                if (x < kGraphEpochBase + 2 || x > kGraphEpochLimit) return fail(PCCL_ERR_INVALID, "test_graph_epoch_limit must be " + std::to_string(kGraphEpochBase + 2) + " .. " + std::to_string(kGraphEpochLimit));
                ctx->graph_epoch_limit = (int32_t)x;
            }
        }
        else if (k == "check_races") { ctx->check_races = int_value(k, value) != 0; relink = true; }
        else if (k == "vecs_per_thread") {
            int u = int_value(k, value);
            if (u != 1 && u != 2 && u != 4) return fail(PCCL_ERR_INVALID, "vecs_per_thread must be 1, 2 or 4");
            ctx->vecs_per_thread = u; relink = true;
        }
        else if (k == "slot_store_waves") {
            const int v = int_value(k, value);
            if (v < -1 || v > 1) return fail(PCCL_ERR_INVALID, "slot_store_waves must be -1 (automatic), 0 or 1");
            ctx->slot_store_waves = v;
        }
        else if (k == "level_graph") ctx->level_graph = int_value(k, value) != 0;
        else if (k == "phased") {
            const int x = int_value(k, value);
            if (x < -1 || x > 1) return fail(PCCL_ERR_INVALID, "phased must be -1 (automatic), 0 or 1");
            ctx->phased = x;
        }
        else if (k == "phased_shape") {
            const int x = int_value(k, value);
            if (x < -1 || x > 1) return fail(PCCL_ERR_INVALID, "phased_shape must be -1 (automatic), 0 (512 threads x 16 vectors) or 1 (256 x 32)");
            ctx->phased_shape = x;
        }
        else if (k == "phased_sweeps") {
            const int x = int_value(k, value);
            if (x != -1 && x != 1 && x != 2) return fail(PCCL_ERR_INVALID, "phased_sweeps must be -1 (automatic), 1 or 2");
            ctx->phased_sweeps = x;
        }
        else if (k == "phased_linear") {
            const int x = int_value(k, value);
            if (x < -1 || x > 1) return fail(PCCL_ERR_INVALID, "phased_linear must be -1 (automatic), 0 or 1");
            ctx->phased_linear = x;
        }
        else if (k == "phased_exchange") {
            const int x = int_value(k, value);
            if (x < -1 || x > 1) return fail(PCCL_ERR_INVALID, "phased_exchange must be -1 (automatic), 0 or 1");
            ctx->phased_exchange = x;
        }
        else if (k == "phased_barriers") ctx->phased_barriers = int_value(k, value) != 0;
        else if (k == "phased_timeout_us") { ctx->phased_timeout_us = int_value(k, value); if (ctx->phased_timeout_us < 0) ctx->phased_timeout_us = 0; }
        else if (k == "lds_slots") { ctx->lds_slots = int_value(k, value) != 0; relink = true; }
        else if (k == "slot_direct" || k == "slot_threads" || k == "slot_vecs") {
            // checked against the shape linking would choose with the new value in place
            int threads = ctx->slot_threads, vecs = ctx->slot_vecs;
            bool direct = ctx->slot_direct;
            const int x = int_value(k, value);
            if (k == "slot_threads") {
                if (x != 0 && x != 64 && x != 128 && x != 256 && x != 512 && x != 1024) return fail(PCCL_ERR_INVALID, "slot_threads must be 0 (automatic), 64, 128, 256, 512 or 1024");
                threads = x;
            } else if (k == "slot_vecs") {
                if (x != 0 && x != 1 && x != 2 && x != 4) return fail(PCCL_ERR_INVALID, "slot_vecs must be 0 (automatic), 1, 2 or 4");
                vecs = x;
            } else direct = x != 0;
            if (!direct && vecs > 1) return fail(PCCL_ERR_INVALID, "slot_vecs above 1 needs slot_direct=1 (first touches fetched through registers take one vector per thread)");
            const std::string why = slot_shape_error(ctx->R, slot_shape(ctx->R, threads, vecs, direct));
            if (!why.empty()) return fail(PCCL_ERR_INVALID, why);
            ctx->slot_threads = threads; ctx->slot_vecs = vecs; ctx->slot_direct = direct; relink = true;
        }
        else if (k == "slot_lds_kib") {
            int b = int_value(k, value);
            if (b < 0 || b > 160) return fail(PCCL_ERR_INVALID, "slot_lds_kib must be 0 (automatic) to 160");
            ctx->slot_lds_kib = b; relink = true;
        }
        else if (k == "step_tile_bytes") {
            int64_t b = whole_number(k, value);
            if (b < 0 || b % 4096) return fail(PCCL_ERR_INVALID, "step_tile_bytes must be 0 (automatic) or a positive multiple of 4096");
            ctx->step_tile_bytes = b; relink = true;
        } else return fail(PCCL_ERR_INVALID, "unknown option '" + k + "'");
        if (relink) {
            HIP_TRY(hipSetDevice(ctx->device));
            HIP_TRY(hipDeviceSynchronize());
            for (auto& kv : ctx->ops) kv.second.release();
        }
        return 0;
    });
}

int pccl_hip_get_option(pccl_hip_ctx* ctx, const char* key, char* value, size_t cap) {
    return guarded([&] {
        if (!ctx || !key || !value || cap == 0) return fail(PCCL_ERR_INVALID, "null argument");
        std::lock_guard<std::mutex> lock(ctx->mu);
        const std::string k = key;
        std::string v;
        if (k == "mode") v = ctx->mode == Mode::Auto ? "auto" : ctx->mode == Mode::Column ? "column" : ctx->mode == Mode::Stepwise ? "stepwise" : "persistent";
        else if (k == "num_blocks") v = std::to_string(ctx->num_blocks);
        else if (k == "timing") v = std::to_string((int)ctx->timing);
        else if (k == "trace_ranges") v = std::to_string((int)ctx->trace_ranges);
        else if (k == "fuse_staging") v = std::to_string((int)ctx->fuse_staging);
        else if (k == "wait_timeout_ms") v = std::to_string(ctx->wait_timeout_ms);
        else if (k == "check_races") v = std::to_string((int)ctx->check_races);
        else if (k == "test_host_epoch_limit") v = std::to_string(ctx->host_epoch_limit);
        else if (k == "test_graph_epoch_limit") v = std::to_string(ctx->graph_epoch_limit);
        else if (k == "vecs_per_thread") v = std::to_string(ctx->vecs_per_thread);
        else if (k == "slot_direct") v = std::to_string((int)ctx->slot_direct);
        else if (k == "slot_store_waves") v = std::to_string(ctx->slot_store_waves);
        else if (k == "level_graph") v = std::to_string((int)ctx->level_graph);
        else if (k == "phased") v = std::to_string(ctx->phased);
        else if (k == "phased_shape") v = std::to_string(ctx->phased_shape);
        else if (k == "phased_exchange") v = std::to_string(ctx->phased_exchange);
        else if (k == "phased_sweeps") v = std::to_string(ctx->phased_sweeps);
        else if (k == "phased_linear") v = std::to_string(ctx->phased_linear);
        else if (k == "phased_barriers") v = std::to_string((int)ctx->phased_barriers);
        else if (k == "phased_timeout_us") v = std::to_string(ctx->phased_timeout_us);
        else if (k == "lds_slots") v = std::to_string((int)ctx->lds_slots);
        else if (k == "slot_threads") v = std::to_string(ctx->slot_threads);
        else if (k == "slot_vecs") v = std::to_string(ctx->slot_vecs);
        else if (k == "slot_lds_kib") v = std::to_string(ctx->slot_lds_kib);
        else if (k == "step_tile_bytes") v = std::to_string(ctx->step_tile_bytes);
        else if (k == "num_vranks") v = std::to_string(ctx->R);
        else if (k == "signals") {   // the semaphores above zero, "rank:id=count" joined by commas, ordered by (rank, id)
            for (const auto& kv : ctx->signals)
                v += (v.empty() ? "" : ",") + std::to_string(kv.first.first) + ":" + std::to_string(kv.first.second) + "=" + std::to_string(kv.second);
        }
        else if (k.rfind("runner_inplace:", 0) == 0 || k.rfind("runner_staged:", 0) == 0) {
            // which kernel an execution of that operation would launch now, given its plan, the tensors'
            // size and the options (16-byte aligned, non-overlapping tensors assumed)
            const bool staged = k[7] == 's';
            OpEntry& e = find_entry(ctx, k.c_str() + (staged ? 14 : 15));
            HIP_TRY(hipSetDevice(ctx->device));
            refresh_link(ctx, e, nullptr, false);
            link_entry(ctx, e);
            const Program& P = e.prog;
            const bool column_ok = ctx->mode == Mode::Auto || ctx->mode == Mode::Column;
            if (staged && P.collective_type == "alltoall" && ctx->fuse_staging && e.gather.p && ctx->mode == Mode::Auto) v = "gather_kernel";
            else if (staged && !(ctx->fuse_staging && column_ok && P.position_aligned && !P.direct_segs.empty()))
                v = std::string("staging + ") + (ctx->mode == Mode::Persistent ? "persistent_kernel" : (P.position_aligned && column_ok) ? "column" : "level_kernel");
            else if (!column_ok || !P.position_aligned) v = ctx->mode == Mode::Persistent ? "persistent_kernel" : "level_kernel";
            else if (wants_phased(ctx, e, staged)) v = "phased_kernel";
            else v = e.slot_threads > 0 ? "column_slot_kernel" : "column_kernel";
        }
        else if (k.rfind("phased_shape_inplace:", 0) == 0 || k.rfind("phased_shape_staged:", 0) == 0) {
            // the shape of the phased runner an execution of that operation would use now, as
            // "shape=N group=K meetings=M", or "none" if it would not run there
            const bool staged = k[13] == 's';
            OpEntry& e = find_entry(ctx, k.c_str() + (staged ? 20 : 21));
            HIP_TRY(hipSetDevice(ctx->device));
            refresh_link(ctx, e, nullptr, false);
            link_entry(ctx, e);
            const bool column_ok = ctx->mode == Mode::Auto || ctx->mode == Mode::Column;
            const bool plan = e.prog.position_aligned && column_ok && (!staged || (ctx->fuse_staging && !e.prog.direct_segs.empty()));
            if (!plan || !wants_phased(ctx, e, staged)) v = "none";
            else {
                const PhasedLaunch L = phased_launch_for(ctx, e, staged);
                v = "shape=" + std::to_string(L.shape) + " group=" + std::to_string(L.group) + (L.group_segs > 1 ? " segments=" + std::to_string(L.group_segs) : std::string()) + " meetings=" + std::to_string(L.barriers);
            }
        }
        else if (k.rfind("slot_shape:", 0) == 0) {
            // the slot runner's workgroup for that operation as linked now: "threads x vectors", "0x0" if
            // its column plan runs on the register runner or it has none
            OpEntry& e = find_entry(ctx, k.c_str() + 11);
            HIP_TRY(hipSetDevice(ctx->device));
            refresh_link(ctx, e, nullptr, false);
            link_entry(ctx, e);
            v = e.slot_threads > 0 ? std::to_string(e.slot_threads) + "x" + std::to_string(e.slot_vecs) : "0x0";
        }
        else return fail(PCCL_ERR_INVALID, "unknown option '" + k + "'");
        if (v.size() + 1 > cap) return fail(PCCL_ERR_INVALID, "value buffer too small");
        std::memcpy(value, v.c_str(), v.size() + 1);
        return 0;
    });
}

int pccl_hip_execute(pccl_hip_ctx* ctx, const char* name, const void* const* inputs, void* const* outputs,
                     size_t in_bytes, size_t out_bytes, void* stream, int sync) {
    return guarded([&] {
        if (!ctx || !inputs || !outputs) return fail(PCCL_ERR_INVALID, "null argument");
        std::lock_guard<std::mutex> lock(ctx->mu);
        HIP_TRY(hipSetDevice(ctx->device));
        OpEntry& e = find_entry(ctx, name);
        hipStream_t s = (hipStream_t)stream;
        refresh_link(ctx, e, s, true);
        link_entry(ctx, e, s, true);
        for (int r = 0; r < ctx->R; ++r)
            if (!inputs[r] || !outputs[r]) return fail(PCCL_ERR_INVALID, "null tensor for virtual rank " + std::to_string(r));
        // on the caller's tensors where the program allows it, else through the rank buffers
        if (!run_direct(ctx, e, inputs, outputs, in_bytes, out_bytes, s) &&
            !run_gather(ctx, e, inputs, outputs, in_bytes, out_bytes, s))
            run_staged(ctx, e, inputs, outputs, in_bytes, out_bytes, s);
        commit_signals(ctx, e);
        ctx->last_stream = s;
        if (sync) { HIP_TRY(hipStreamSynchronize(s)); check_stall(e, name); }
        return 0;
    });
}

int pccl_hip_execute_inplace(pccl_hip_ctx* ctx, const char* name, void* const* bufs, size_t buf_bytes,
                             void* stream, int sync) {
    return guarded([&] {
        if (!ctx || !bufs) return fail(PCCL_ERR_INVALID, "null argument");
        std::lock_guard<std::mutex> lock(ctx->mu);
        HIP_TRY(hipSetDevice(ctx->device));
        OpEntry& e = find_entry(ctx, name);
        hipStream_t s = (hipStream_t)stream;
        refresh_link(ctx, e, s, true);
        link_entry(ctx, e, s, true);
        {
            TraceRange exe(ctx->trace_ranges, "execute");
            run_program(ctx, e, (char* const*)bufs, buf_bytes, s);
        }
        commit_signals(ctx, e);
        ctx->last_stream = s;
        if (sync) { HIP_TRY(hipStreamSynchronize(s)); check_stall(e, name); }
        return 0;
    });
}

int pccl_hip_execute_inplace_static(pccl_hip_ctx* ctx, const char* name, void* const* bufs, size_t buf_bytes,
                                    void* stream, int sync) {
    return guarded([&] {
        if (!ctx || !bufs) return fail(PCCL_ERR_INVALID, "null argument");
        std::lock_guard<std::mutex> lock(ctx->mu);
        HIP_TRY(hipSetDevice(ctx->device));
        OpEntry& e = find_entry(ctx, name);
        hipStream_t s = (hipStream_t)stream;
        refresh_link(ctx, e, s, true, false);            // never frees device memory here
        link_host(ctx, e);                               // host memory only
        const Program& P = e.prog;
        StaticWorkspace& ws = static_ws(ctx->device);
        std::lock_guard<std::mutex> wlock(ws.mu);
        if (!ws.ptr) return fail(PCCL_ERR_HIP, "the static workspace of this GPU has no address");
        const StaticLayout lay = static_layout(P);
        if (lay.total > ws.bytes)
            return fail(PCCL_ERR_INVALID, "operation '" + std::string(name) + "' needs " + std::to_string(lay.total) + " bytes of runner tables (" +
                                              std::to_string(P.num_items) + " work items, " + std::to_string(P.ops.size()) + " data ops); the static workspace holds " +
                                              std::to_string(ws.bytes) + ": use pccl_hip_execute_inplace, or larger work items (option step_tile_bytes)");
        const size_t es = elem_size(P.dtype);
        if ((size_t)P.buffer_elems * es > buf_bytes)
            return fail(PCCL_ERR_INVALID, "rank buffers of " + std::to_string(buf_bytes) + " bytes are smaller than the " + std::to_string((size_t)P.buffer_elems * es) + " bytes the graph addresses");
        RankPtrs ptrs;
        std::memset(&ptrs, 0, sizeof(ptrs));
        for (int r = 0; r < ctx->R; ++r) {
            if (!bufs[r]) return fail(PCCL_ERR_INVALID, "null rank buffer " + std::to_string(r));
            if ((uintptr_t)bufs[r] % es) return fail(PCCL_ERR_INVALID, "rank buffer " + std::to_string(r) + " is not aligned to the element size");
            ptrs.p[r] = (char*)bufs[r];
            ptrs.p[PCCL_HIP_MAX_VRANKS + r] = (char*)bufs[r];
        }
        if (P.ops.empty()) return 0;
        const bool capturing = is_capturing(s);
        int rc = 0;
        if (ws.owner != e.generation || ws.epoch >= ctx->host_epoch_limit) {
            // the workspace holds another operation's tables (or nothing, or the launch numbers have run
            // out): clear the progress block and write this operation's tables, all by kernels on `s`
            if (capturing)
                return fail(PCCL_ERR_INVALID, "the stream is capturing and the static workspace does not hold this operation's tables: "
                                              "execute it once outside the capture first");
            rc = launch_fill_zero(ws.ptr, lay.ops, s);   // a fill kernel, not a memset node (the block, the flags, the ready words)
            if (!rc) rc = launch_table_write(e.host.step_ops.data(), e.host.step_ops.size() * sizeof(DevStepOp), ws.ptr + lay.ops, s);
            if (!rc) rc = launch_table_write(e.host.step_deps_padded.data(), e.host.step_deps_padded.size() * sizeof(int32_t), ws.ptr + lay.deps, s);
            if (!rc) rc = launch_item_op_fill((const DevStepOp*)(ws.ptr + lay.ops), (int)P.ops.size(), (int32_t*)(ws.ptr + lay.item_op), s);
            // last: the block now belongs to this operation (StepState::owner, and a zero launch counter beside it)
            const uint64_t head = static_tag(e);
            if (!rc) rc = launch_table_write(&head, sizeof(head), ws.ptr, s);
            if (rc) { ws.owner = 0; return fail(PCCL_ERR_HIP, std::string("writing the runner tables: ") + hipGetErrorString((hipError_t)rc)); }
            ws.owner = e.generation;
            ws.epoch = 0;
        }
        StepwiseLaunch L{};
        L.ops = (const DevStepOp*)(ws.ptr + lay.ops); L.num_ops = (int)P.ops.size();
        L.deps = (const int32_t*)(ws.ptr + lay.deps); L.item_op = (const int32_t*)(ws.ptr + lay.item_op);
        L.num_items = (int)P.num_items; L.tile_elems = P.tile_elems; L.state = (StepState*)ws.ptr;
        L.dtype = P.dtype; L.num_blocks = ctx->num_blocks;
        L.epoch = capturing ? 0 : ++ws.epoch;            // recorded launches take their number from the device-side counter
        L.owner_tag = static_tag(e);                     // a replay that finds another operation's tables does nothing
        L.graph_epoch_limit = ctx->graph_epoch_limit;
        L.timeout_ticks = (uint64_t)ctx->wait_timeout_ms * 100000ull;
        {
            TraceRange exe(ctx->trace_ranges, "execute"), range(ctx->trace_ranges, "executor_kernel");
            rc = launch_persistent(L, ptrs, s);
        }
        if (rc) { ws.owner = 0; return fail(PCCL_ERR_HIP, std::string("kernel launch failed: ") + hipGetErrorString((hipError_t)rc)); }
        commit_signals(ctx, e);
        e.ran_static = true;
        ctx->last_stream = s;
        if (sync) {
            HIP_TRY(hipStreamSynchronize(s));
            e.ran_static = false;
            read_static_block(ctx, ws, name);
        }
        return 0;
    });
}

int pccl_hip_sync(pccl_hip_ctx* ctx, const char* name) {
    return guarded([&] {
        if (!ctx) return fail(PCCL_ERR_INVALID, "null argument");
        std::lock_guard<std::mutex> lock(ctx->mu);
        auto it = ctx->ops.find(name ? name : "");
        if (it == ctx->ops.end()) return 0;  // the reference returns silently
        HIP_TRY(hipSetDevice(ctx->device));
        HIP_TRY(hipStreamSynchronize(ctx->last_stream));
        check_stall(it->second, it->first);
        check_stall_static(ctx, it->second, it->first);
        return 0;
    });
}

int pccl_hip_reset_signals(pccl_hip_ctx* ctx, const char* name) {
    return guarded([&] {
        if (!ctx) return fail(PCCL_ERR_INVALID, "null argument");
        std::lock_guard<std::mutex> lock(ctx->mu);
        auto it = ctx->ops.find(name ? name : "");
        if (it == ctx->ops.end()) return 0;
        HIP_TRY(hipSetDevice(ctx->device));
        HIP_TRY(hipStreamSynchronize(ctx->last_stream));
        // The reference clears the engine's whole signal region, whichever operation is named
        // (csrc/engine_c.cc:576-593): every carried count goes.  Operations that were linked for other
        // counts are linked again when they are next executed.  What else can be left over is the
        // runner's progress block after an aborted launch.
        ctx->signals.clear();
        OpEntry& e = it->second;
        if (e.linked && e.state.p) {
            int rc = launch_fill_zero(e.state.p, e.state.bytes, ctx->last_stream);
            if (rc) return fail(PCCL_ERR_HIP, hipGetErrorString((hipError_t)rc));
            HIP_TRY(hipStreamSynchronize(ctx->last_stream));
            e.epoch = 0;
        }
        return 0;
    });
}

int pccl_hip_op_info(pccl_hip_ctx* ctx, const char* name, pccl_program_info* out) {
    return guarded([&] {
        if (!ctx || !out) return fail(PCCL_ERR_INVALID, "null argument");
        std::lock_guard<std::mutex> lock(ctx->mu);
        HIP_TRY(hipSetDevice(ctx->device));
        OpEntry& e = find_entry(ctx, name);
        refresh_link(ctx, e, nullptr, false);
        link_host(ctx, e);      // inspection needs no device memory
        fill_info(e.prog, out);
        if (e.slot_threads > 0) {   // the traffic of the runner this context would launch
            out->column_load_bytes = e.prog.slot_load_bytes;
            out->column_store_bytes = e.prog.slot_store_bytes;
            out->staged_load_bytes = e.prog.direct_slot_load_bytes;
            out->staged_store_bytes = e.prog.direct_slot_store_bytes;
        }
        return 0;
    });
}

int pccl_hip_last_kernel_ms(pccl_hip_ctx* ctx, const char* name, float* ms) {
    return guarded([&] {
        if (!ctx || !ms) return fail(PCCL_ERR_INVALID, "null argument");
        std::lock_guard<std::mutex> lock(ctx->mu);
        OpEntry& e = find_entry(ctx, name);
        if (!e.timed) return fail(PCCL_ERR_INVALID, "no timed launch: set option timing=1 and execute first");
        HIP_TRY(hipEventSynchronize(e.ev1));
        HIP_TRY(hipEventElapsedTime(ms, e.ev0, e.ev1));
        return 0;
    });
}

int pccl_hip_reduce(int dtype, int redop, const void* a, const void* b, void* c, size_t n, void* stream) {
    return guarded([&] {
        if (!a || !b || !c) return fail(PCCL_ERR_INVALID, "null argument");
        if (dtype < PCCL_F32 || dtype > PCCL_I32) return fail(PCCL_ERR_UNSUPPORTED, "unknown dtype");
        if (redop < PCCL_SUM || redop > PCCL_MIN) return fail(PCCL_ERR_INVALID, "bad reduce operator");
        int es = elem_size(dtype);
        if ((uintptr_t)a % es || (uintptr_t)b % es || (uintptr_t)c % es) return fail(PCCL_ERR_INVALID, "pointers must be aligned to the element size");
        int rc = launch_reduce(dtype, redop, a, b, c, n, stream);
        if (rc) return fail(PCCL_ERR_HIP, hipGetErrorString((hipError_t)rc));
        return 0;
    });
}

int pccl_hip_copy(int dtype, const void* src, void* dst, size_t n, void* stream) {
    return guarded([&] {
        if (!src || !dst) return fail(PCCL_ERR_INVALID, "null argument");
        int es = elem_size(dtype);
        if (!es) return fail(PCCL_ERR_INVALID, "bad dtype");
        int rc = launch_copy_bytes(src, dst, n * es, stream);
        if (rc) return fail(PCCL_ERR_HIP, hipGetErrorString((hipError_t)rc));
        return 0;
    });
}

}  // extern "C"
