// One rank's graph as the executor sees it: triggers + dependency metadata.
#pragma once

#include <cstdint>
#include <string>
#include <vector>

#include "../../include/pccl_hip.h"

namespace pccl_hip {

struct Error {
    int code;
    std::string msg;
};

enum class OpKind : int { Noop = 0, Reduce = 1, Copy = 2, Notify = 3, Wait = 4 };

struct GraphOp {
    OpKind kind = OpKind::Noop;
    int primitive_type = 0;  // reference id (primitive_config.h) or extension id
    int redop = PCCL_SUM;
    int index = 0;           // label from the document
    int channel = 0;
    int peer = 0;            // data: source rank; notify: target; wait: source (unused at run time)
    int64_t off0 = 0, off1 = 0, off2 = 0, size = 0;  // elements; signals: off0 = signal id
    std::vector<int> deps;   // positions in RankGraph::ops
    std::vector<int> nexts;  // positions in RankGraph::ops (at most 8, like the reference)
    int num_deps_declared = 0;
};

struct RankGraph {
    std::vector<GraphOp> ops;
    int dtype = PCCL_F32;
    bool has_dtype = false;
    int64_t tensor_elems = 0;
    std::string collective_type;

    int64_t max_extent() const;  // max(offset + size) over data ops
};

int dtype_from_name(const std::string& name);  // -1 if unknown
int elem_size(int dtype);

// Throws Error.
RankGraph load_graph_json(const char* text, size_t len);
RankGraph load_graph_file(const std::string& path);
RankGraph graph_from_triggers(const pccl_trigger* trig, const pccl_primitive_meta* meta, int n,
                              const char* collective_type);

void graph_to_triggers(const RankGraph& g, std::vector<pccl_trigger>* trig,
                       std::vector<pccl_primitive_meta>* meta);

// Returns false when the graph is not a set of per-channel linear chains the fused runner accepts.
bool build_fused_steps(const RankGraph& g, std::vector<pccl_fused_step>* steps,
                       std::vector<int>* channel_offsets);

}  // namespace pccl_hip
