// Graph loading (JSON v2 -> triggers) and fused-step grouping.
#include "graph.h"

#include <algorithm>
#include <cstring>
#include <fstream>
#include <sstream>

#include "json_min.h"

namespace pccl_hip {

int dtype_from_name(const std::string& name) {
    if (name == "float32") return PCCL_F32;
    if (name == "float16") return PCCL_F16;
    if (name == "bfloat16") return PCCL_BF16;
    if (name == "float8_e4m3") return PCCL_F8E4M3;
    if (name == "float8_e5m2") return PCCL_F8E5M2;
    if (name == "int32") return PCCL_I32;
    return -1;
}

int elem_size(int dtype) {
    switch (dtype) {
        case PCCL_F32: case PCCL_I32: return 4;
        case PCCL_F16: case PCCL_BF16: return 2;
        case PCCL_F8E4M3: case PCCL_F8E5M2: return 1;
        default: return 0;
    }
}

int64_t RankGraph::max_extent() const {
    int64_t m = 0;
    for (auto& o : ops) {
        if (o.kind == OpKind::Reduce)
            m = std::max({m, o.off0 + o.size, o.off1 + o.size, o.off2 + o.size});
        else if (o.kind == OpKind::Copy)
            m = std::max({m, o.off0 + o.size, o.off1 + o.size});
    }
    return m;
}

namespace {

int reduce_ptype(int dtype, bool tma) {
    if (dtype == PCCL_I32) return PCCL_PT_REDUCE_I32;
    return (tma ? PCCL_PT_TMA_REDUCE_F32 : PCCL_PT_REDUCE_F32) + dtype;
}
int copy_ptype(int dtype, bool tma) {
    if (dtype == PCCL_I32) return PCCL_PT_COPY_I32;
    return (tma ? PCCL_PT_TMA_COPY_F32 : PCCL_PT_COPY_F32) + dtype;
}

int redop_from_name(const std::string& s) {
    if (s == "sum") return PCCL_SUM;
    if (s == "max") return PCCL_MAX;
    if (s == "min") return PCCL_MIN;
    return -1;
}

// Which executors this plugin runs.  The reference maps "cuda_*" to its device plugin and "host"
// to the host plugin (csrc/engine/graph_builder.cc:48-58); only SM primitives and the TMA
// primitives' SM fallback exist here.
void check_executor(const std::string& ex, const std::string& prim) {
    if (ex == "cuda_sm" || ex == "cuda_tma") return;
    throw Error{PCCL_ERR_UNSUPPORTED, "executor '" + ex + "' (primitive '" + prim +
                                          "') is not provided by the HIP plugin: only cuda_sm and "
                                          "cuda_tma (run as SM copy/reduce) are"};
}

int64_t param_int(const json::Value& params, const char* key, const std::string& prim) {
    const json::Value* v = params.find(key);
    if (!v) throw Error{PCCL_ERR_PARSE, "primitive '" + prim + "' lacks params." + key};
    return v->as_int(key);
}

void check_i32(int64_t v, const char* what) {
    if (v < 0 || v > INT32_MAX)
        throw Error{PCCL_ERR_PARSE, std::string(what) + " out of the 32-bit element range"};
}

}  // namespace

RankGraph load_graph_json(const char* text, size_t len) {
    json::Value doc;
    try {
        doc = json::parse(text, len);
    } catch (const json::ParseError& e) {
        throw Error{PCCL_ERR_PARSE, e.what()};
    }
    if (!doc.is_object() || !doc.contains("operations") || !doc.at("operations").is_array())
        throw Error{PCCL_ERR_NOT_A_GRAPH, "graph document has no 'operations' array"};

    RankGraph g;
    std::string dtype_name;
    if (const json::Value* ti = doc.find("tensor_info")) {
        if (const json::Value* d = ti->find("dtype")) {
            dtype_name = d->as_string("tensor_info.dtype");
            int dt = dtype_from_name(dtype_name);
            if (dt >= 0) { g.dtype = dt; g.has_dtype = true; }
        }
        if (const json::Value* sh = ti->find("shape")) {
            int64_t n = 1;
            if (sh->is_array()) for (auto& d : sh->arr) n *= d.as_int("tensor_info.shape");
            g.tensor_elems = n;
        }
    }
    if (const json::Value* ct = doc.find("collective_type")) g.collective_type = ct->as_string("collective_type");

    const auto& ops = doc.at("operations").arr;
    g.ops.resize(ops.size());
    // `index` values label ops; dependencies / next_ops refer to them.  The emitter writes
    // index == position, but resolve through a map so a reordered document still links.
    std::vector<std::pair<int64_t, int>> by_index;
    try {
        for (size_t pos = 0; pos < ops.size(); ++pos) {
            const json::Value& op = ops[pos];
            if (!op.is_object() || !op.contains("index") || !op.contains("executor") || !op.contains("primitive"))
                throw Error{PCCL_ERR_NOT_A_GRAPH, "operation " + std::to_string(pos) + " lacks index/executor/primitive"};
            GraphOp& o = g.ops[pos];
            o.index = (int)op.at("index").as_int("index");
            by_index.emplace_back(o.index, (int)pos);
            o.channel = (int)op.int_or("channel", 0);
            if (o.channel < 0 || o.channel >= PCCL_HIP_MAX_CHANNELS)
                throw Error{PCCL_ERR_PARSE, "operation " + std::to_string(pos) + ": channel " + std::to_string(o.channel) + " outside 0.." + std::to_string(PCCL_HIP_MAX_CHANNELS - 1)};
            const std::string& prim = op.at("primitive").as_string("primitive");
            const std::string& ex = op.at("executor").as_string("executor");
            static const json::Value empty_obj = [] { json::Value v; v.kind = json::Value::Object; return v; }();
            const json::Value& params = op.contains("params") ? op.at("params") : empty_obj;

            bool is_reduce = prim == "sm.reduce" || prim == "tma.reduce";
            bool is_copy = prim == "sm.copy" || prim == "tma.copy";
            bool tma = prim.rfind("tma.", 0) == 0;
            if (is_reduce || is_copy) {
                check_executor(ex, prim);
                if (!g.has_dtype)
                    throw Error{PCCL_ERR_PARSE, "Unsupported dtype '" + dtype_name + "'"};
                // peer = source_rank, else target_rank, else 0 (sm_channel.h:84)
                const json::Value* pr = params.find("source_rank");
                if (!pr) pr = params.find("target_rank");
                o.peer = pr ? (int)pr->as_int("source_rank") : 0;
                if (is_reduce) {
                    o.kind = OpKind::Reduce;
                    o.primitive_type = reduce_ptype(g.dtype, tma);
                    o.off0 = param_int(params, "remote_offset", prim);
                    o.off1 = param_int(params, "src_offset", prim);
                    o.off2 = param_int(params, "dst_offset", prim);
                    o.size = param_int(params, "count", prim);
                    if (const json::Value* ro = params.find("reduce_op")) {
                        o.redop = redop_from_name(ro->as_string("reduce_op"));
                        if (o.redop < 0)
                            throw Error{PCCL_ERR_UNSUPPORTED, "reduce_op '" + ro->s + "' is not supported (sum, max, min are)"};
                    }
                    check_i32(o.off2, "dst_offset");
                } else {
                    o.kind = OpKind::Copy;
                    o.primitive_type = copy_ptype(g.dtype, tma);
                    o.off0 = param_int(params, "src_offset", prim);
                    o.off1 = param_int(params, "dst_offset", prim);
                    o.size = param_int(params, "size", prim);
                }
                check_i32(o.off0, "offset"); check_i32(o.off1, "offset"); check_i32(o.size, "size");
            } else if (prim == "notify" || prim == "sm.notify") {
                check_executor(ex, prim);
                o.kind = OpKind::Notify;
                o.primitive_type = PCCL_PT_NOTIFY;
                o.peer = (int)param_int(params, "target_rank", prim);
                o.off0 = param_int(params, "signal_id", prim);
            } else if (prim == "wait_notify" || prim == "sm.wait_notify") {
                check_executor(ex, prim);
                o.kind = OpKind::Wait;
                o.primitive_type = PCCL_PT_WAIT_NOTIFY;
                o.peer = (int)param_int(params, "source_rank", prim);
                o.off0 = param_int(params, "signal_id", prim);
            } else if (prim == "noop") {
                o.kind = OpKind::Noop;
                o.primitive_type = PCCL_PT_NOOP;
            } else {
                throw Error{PCCL_ERR_PARSE, "unknown primitive '" + prim + "'"};
            }
            if ((o.kind == OpKind::Notify || o.kind == OpKind::Wait) &&
                (o.off0 < 0 || o.off0 >= PCCL_HIP_NUM_SIGNALS))
                throw Error{PCCL_ERR_PARSE, "signal_id " + std::to_string(o.off0) + " outside 0.." + std::to_string(PCCL_HIP_NUM_SIGNALS - 1)};
        }
        std::sort(by_index.begin(), by_index.end());
        for (size_t k = 1; k < by_index.size(); ++k)
            if (by_index[k].first == by_index[k - 1].first)
                throw Error{PCCL_ERR_PARSE, "duplicate operation index " + std::to_string(by_index[k].first)};
        auto resolve = [&](int64_t idx) -> int {
            auto it = std::lower_bound(by_index.begin(), by_index.end(), std::make_pair(idx, INT32_MIN));
            if (it == by_index.end() || it->first != idx)
                throw Error{PCCL_ERR_PARSE, "reference to unknown operation index " + std::to_string(idx)};
            return it->second;
        };
        for (size_t pos = 0; pos < ops.size(); ++pos) {
            const json::Value& op = ops[pos];
            GraphOp& o = g.ops[pos];
            if (const json::Value* d = op.find("dependencies"))
                for (auto& v : d->arr) o.deps.push_back(resolve(v.as_int("dependencies")));
            o.num_deps_declared = (int)o.deps.size();
            if (const json::Value* n = op.find("next_ops"))
                for (auto& v : n->arr)
                    if (o.nexts.size() < 8) o.nexts.push_back(resolve(v.as_int("next_ops")));  // graph_builder.cc:69
        }
    } catch (const json::ParseError& e) {
        throw Error{PCCL_ERR_PARSE, e.what()};
    }
    return g;
}

RankGraph load_graph_file(const std::string& path) {
    std::ifstream f(path, std::ios::binary);
    if (!f.is_open()) throw Error{PCCL_ERR_NOT_FOUND, "cannot open graph file '" + path + "'"};
    std::stringstream ss;
    ss << f.rdbuf();
    std::string text = ss.str();
    return load_graph_json(text.data(), text.size());
}

namespace {
// dtype / kind of a reference primitive id
bool decode_ptype(int pt, OpKind* kind, int* dtype) {
    auto in = [&](int base) { return pt >= base && pt < base + 5; };
    if (in(PCCL_PT_REDUCE_F32)) { *kind = OpKind::Reduce; *dtype = pt - PCCL_PT_REDUCE_F32; return true; }
    if (in(PCCL_PT_COPY_F32)) { *kind = OpKind::Copy; *dtype = pt - PCCL_PT_COPY_F32; return true; }
    if (in(PCCL_PT_TMA_REDUCE_F32)) { *kind = OpKind::Reduce; *dtype = pt - PCCL_PT_TMA_REDUCE_F32; return true; }
    if (in(PCCL_PT_TMA_COPY_F32)) { *kind = OpKind::Copy; *dtype = pt - PCCL_PT_TMA_COPY_F32; return true; }
    if (pt == PCCL_PT_REDUCE_I32) { *kind = OpKind::Reduce; *dtype = PCCL_I32; return true; }
    if (pt == PCCL_PT_COPY_I32) { *kind = OpKind::Copy; *dtype = PCCL_I32; return true; }
    if (pt == PCCL_PT_NOTIFY) { *kind = OpKind::Notify; *dtype = -1; return true; }
    if (pt == PCCL_PT_WAIT_NOTIFY) { *kind = OpKind::Wait; *dtype = -1; return true; }
    if (pt == PCCL_PT_NOOP) { *kind = OpKind::Noop; *dtype = -1; return true; }
    return false;
}
}  // namespace

RankGraph graph_from_triggers(const pccl_trigger* trig, const pccl_primitive_meta* meta, int n,
                              const char* collective_type) {
    if (!trig || !meta || n < 0) throw Error{PCCL_ERR_INVALID, "null trigger/meta array"};
    RankGraph g;
    if (collective_type) g.collective_type = collective_type;
    g.ops.resize(n);
    for (int i = 0; i < n; ++i) {
        GraphOp& o = g.ops[i];
        int dt = -1;
        if (!decode_ptype(trig[i].primitive_type, &o.kind, &dt))
            throw Error{PCCL_ERR_UNSUPPORTED, "primitive type id " + std::to_string((int)trig[i].primitive_type) + " is not an SM/TMA data op or a signal"};
        o.primitive_type = trig[i].primitive_type;
        if (dt >= 0) {
            if (g.has_dtype && g.dtype != dt) throw Error{PCCL_ERR_PARSE, "mixed element types in one graph"};
            g.dtype = dt; g.has_dtype = true;
        }
        o.index = trig[i].op_index;
        o.peer = trig[i].peer_rank;
        o.off0 = trig[i].offset_0; o.off1 = trig[i].offset_1; o.off2 = trig[i].offset_2;
        o.size = trig[i].size;
        o.redop = PCCL_SUM;  // the reference runtime has no other operator
        // the same ranges the JSON loader enforces: a negative offset or size would make the
        // kernels address memory in front of a rank buffer
        if (o.kind == OpKind::Reduce || o.kind == OpKind::Copy) {
            const std::string where = "op " + std::to_string(i) + ": ";
            if (o.off0 < 0 || o.off1 < 0 || o.size < 0 || (o.kind == OpKind::Reduce && o.off2 < 0))
                throw Error{PCCL_ERR_PARSE, where + "negative offset or size in a data trigger"};
            const int64_t reach = std::max(o.off0, std::max(o.off1, o.kind == OpKind::Reduce ? o.off2 : 0)) + o.size;
            if (reach > INT32_MAX)
                throw Error{PCCL_ERR_PARSE, where + "offset + size out of the 32-bit element range"};
            if (o.kind == OpKind::Copy) o.off2 = 0;   // unused by copies: whatever the array held there
        } else if (o.kind == OpKind::Notify || o.kind == OpKind::Wait) {
            if (o.off0 < 0 || o.off0 >= PCCL_HIP_NUM_SIGNALS)
                throw Error{PCCL_ERR_PARSE, "op " + std::to_string(i) + ": signal_id " + std::to_string(o.off0) + " outside 0.." + std::to_string(PCCL_HIP_NUM_SIGNALS - 1)};
        }
        o.channel = meta[i].channel;
        if (o.channel < 0 || o.channel >= PCCL_HIP_MAX_CHANNELS) throw Error{PCCL_ERR_PARSE, "channel out of range"};
        o.num_deps_declared = meta[i].num_dependencies;
        int nn = std::min(meta[i].num_next_ops, 8);
        for (int k = 0; k < nn; ++k) {
            int nx = meta[i].next_primitive_index[k];
            if (nx < 0 || nx >= n) throw Error{PCCL_ERR_PARSE, "next_primitive_index out of range"};
            o.nexts.push_back(nx);
        }
    }
    // PrimitiveMeta carries only the dependency count; recover the edges from next lists.
    for (int i = 0; i < n; ++i)
        for (int nx : g.ops[i].nexts) g.ops[nx].deps.push_back(i);
    for (int i = 0; i < n; ++i)
        if ((int)g.ops[i].deps.size() != g.ops[i].num_deps_declared)
            throw Error{PCCL_ERR_PARSE, "op " + std::to_string(i) + ": num_dependencies does not match the next-op lists"};
    return g;
}

void graph_to_triggers(const RankGraph& g, std::vector<pccl_trigger>* trig,
                       std::vector<pccl_primitive_meta>* meta) {
    size_t n = g.ops.size();
    if (trig) trig->assign(n, pccl_trigger{});
    if (meta) meta->assign(n, pccl_primitive_meta{});
    for (size_t i = 0; i < n; ++i) {
        const GraphOp& o = g.ops[i];
        pccl_trigger t{};
        t.primitive_type = (int8_t)o.primitive_type;
        t.redop = (int8_t)o.redop;
        t.op_index = o.index;
        t.peer_rank = o.peer;
        t.offset_0 = (int32_t)o.off0; t.offset_1 = (int32_t)o.off1; t.offset_2 = (int32_t)o.off2;
        t.size = (int32_t)o.size;
        if (trig) (*trig)[i] = t;
        if (meta) {
            pccl_primitive_meta m{};
            m.op_seq_index = o.index;
            m.num_next_ops = (int)o.nexts.size();
            m.num_dependencies = o.num_deps_declared;
            for (size_t k = 0; k < o.nexts.size(); ++k) m.next_primitive_index[k] = o.nexts[k];
            m.device_type = 1;
            m.channel = o.channel;
            std::memcpy(m.params, &t, sizeof(m.params));
            (*meta)[i] = m;
        }
    }
}

bool build_fused_steps(const RankGraph& g, std::vector<pccl_fused_step>* steps,
                       std::vector<int>* channel_offsets) {
    steps->clear();
    channel_offsets->clear();
    int n = (int)g.ops.size();
    if (n == 0) return false;
    int num_ch = 1;
    for (auto& o : g.ops) {
        if (o.num_deps_declared > 1 || o.nexts.size() > 1) return false;
        num_ch = std::max(num_ch, o.channel + 1);
    }
    // chains start at ops without dependencies and follow the single successor
    std::vector<std::vector<int>> chains(num_ch);
    int in_chains = 0;
    for (int i = 0; i < n; ++i) {
        if (g.ops[i].num_deps_declared != 0) continue;
        int c = g.ops[i].channel;
        for (int cur = i; cur >= 0; cur = g.ops[cur].nexts.empty() ? -1 : g.ops[cur].nexts[0]) {
            chains[c].push_back(cur);
            if (++in_chains > n) return false;  // malformed successor lists
        }
    }
    if (in_chains != n) return false;

    auto is_signal = [&](int i) { return g.ops[i].kind == OpKind::Notify || g.ops[i].kind == OpKind::Wait; };
    auto put_data = [&](pccl_fused_step& s, const GraphOp& o) {
        s.primitive_type = (int8_t)o.primitive_type;
        s.peer_rank = o.peer;
        s.offset_0 = (int32_t)o.off0; s.offset_1 = (int32_t)o.off1; s.offset_2 = (int32_t)o.off2;
        s.size = (int32_t)o.size;
    };
    for (int c = 0; c < num_ch; ++c) {
        channel_offsets->push_back((int)steps->size());
        const auto& ch = chains[c];
        size_t pos = 0;
        while (pos < ch.size()) {
            if ((int)steps->size() >= PCCL_HIP_MAX_FUSED_STEPS) return false;
            pccl_fused_step s{};
            const GraphOp& head = g.ops[ch[pos]];
            if (head.kind == OpKind::Notify) {
                s.has_notify = 1; s.notify_peer_rank = head.peer; s.notify_signal_id = (int32_t)head.off0;
                ++pos;
                if (pos < ch.size() && g.ops[ch[pos]].kind == OpKind::Wait) {
                    s.has_wait = 1; s.wait_peer_rank = g.ops[ch[pos]].peer; s.wait_signal_id = (int32_t)g.ops[ch[pos]].off0;
                    ++pos;
                }
                if (pos < ch.size() && !is_signal(ch[pos])) { put_data(s, g.ops[ch[pos]]); ++pos; }
            } else if (head.kind == OpKind::Wait) {
                s.has_wait = 1; s.wait_peer_rank = head.peer; s.wait_signal_id = (int32_t)head.off0;
                ++pos;
                if (pos < ch.size() && !is_signal(ch[pos])) { put_data(s, g.ops[ch[pos]]); ++pos; }
                if (pos < ch.size() && g.ops[ch[pos]].kind == OpKind::Notify) {
                    s.has_notify = 1; s.notify_peer_rank = g.ops[ch[pos]].peer; s.notify_signal_id = (int32_t)g.ops[ch[pos]].off0;
                    ++pos;
                }
            } else {
                return false;  // a step may not open with a data op
            }
            steps->push_back(s);
        }
    }
    channel_offsets->push_back((int)steps->size());
    return true;
}

}  // namespace pccl_hip
