/*
 * pccl_hip.h — C ABI of the MI355X (gfx950) executor plugin for PCCL's SM data path.
 *
 * One process, one GPU.  The R ranks of a schedule are R "virtual ranks": R rank buffers in this
 * GPU's HBM, R per-rank graphs, R semaphore arrays folded into one linked program.  Each entry
 * point names the reference interface it stands in for.  No C++ or torch types cross this
 * boundary: plain pointers, sizes and ints.  Every function returns 0 on success or a negative
 * pccl_status; the message of the last failure on the calling thread is pccl_hip_last_error().
 */
#ifndef PCCL_HIP_H_
#define PCCL_HIP_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define PCCL_HIP_MAX_VRANKS 64
#define PCCL_HIP_MAX_CHANNELS 8     /* reference include/common/config.h:27 */
#define PCCL_HIP_NUM_SIGNALS 4096   /* reference include/common/config.h:24 (ints per rank) */
#define PCCL_HIP_MAX_FUSED_STEPS 128 /* reference include/common/config.h:28 */
#define PCCL_HIP_STATIC_WORKSPACE_BYTES (4u << 20) /* device memory pccl_hip_execute_inplace_static works in, per GPU */

typedef enum {
    PCCL_OK = 0,
    PCCL_ERR_INVALID = -1,     /* bad argument */
    PCCL_ERR_NOT_FOUND = -2,   /* unknown operation name / missing file */
    PCCL_ERR_PARSE = -3,       /* malformed graph document, unknown primitive or dtype */
    PCCL_ERR_LINK = -4,        /* ranks missing, deadlock, unbalanced signals, data race */
    PCCL_ERR_HIP = -5,         /* a HIP runtime call failed */
    PCCL_ERR_UNSUPPORTED = -6, /* valid request this build does not implement */
    PCCL_ERR_NOT_A_GRAPH = -7  /* a readable JSON document without an 'operations' array, or with an
                                * operation lacking index / executor / primitive: the two cases in which
                                * the reference's loader returns false (csrc/engine/graph_builder.cc:22-41) */
} pccl_status;

/* Element types, numbered like the reference's DataType (csrc/plugins/cuda/kernel/compute.h:13-19);
 * PCCL_I32 is an extension (the reference rejects integer dtypes). */
typedef enum { PCCL_F32 = 0, PCCL_F16 = 1, PCCL_BF16 = 2, PCCL_F8E4M3 = 3, PCCL_F8E5M2 = 4, PCCL_I32 = 5 } pccl_dtype;

/* Reduction operators.  The reference runtime always sums; MAX / MIN honour the graph's
 * params.reduce_op and are an extension. */
typedef enum { PCCL_SUM = 0, PCCL_MAX = 1, PCCL_MIN = 2 } pccl_redop;

/* Primitive type ids: reference csrc/plugins/cuda/kernel/primitive_config.h:7-57. */
enum {
    PCCL_PT_NOOP = 0,
    PCCL_PT_REDUCE_F32 = 1,      /* +dtype 0..4 */
    PCCL_PT_COPY_F32 = 6,        /* +dtype 0..4 */
    PCCL_PT_WAIT_NOTIFY = 21,
    PCCL_PT_NOTIFY = 22,
    PCCL_PT_TMA_COPY_F32 = 28,   /* +dtype 0..4: executed as plain copy (the reference's SM fallback) */
    PCCL_PT_TMA_REDUCE_F32 = 33, /* +dtype 0..4: executed as plain reduce */
    PCCL_PT_REDUCE_I32 = 64,     /* extension ids, outside the reference's table */
    PCCL_PT_COPY_I32 = 65
};

/* 32-byte trigger, field offsets of the reference's OpProxyTriggerCudaHandle /
 * SignalProxyTriggerCudaHandle (csrc/plugins/cuda/kernel/proxy_trigger.h:8-30):
 * data ops: offset_0/1/2 = remote/src/dst (reduce) or src/dst/- (copy), size in elements;
 * signals: peer_rank = target (notify) or source (wait), offset_0 = signal id. */
typedef struct {
    int8_t primitive_type;
    int8_t redop;       /* pccl_redop; byte 1 is padding in the reference */
    int8_t pad_[2];
    int32_t op_index;
    int32_t peer_rank;
    int32_t offset_0;
    int32_t offset_1;
    int32_t offset_2;
    int32_t size;
    int32_t reserved_;
} pccl_trigger;

/* Graph metadata per op: layout of the reference's PrimitiveMeta (include/engine/primitive.h:8-17). */
typedef struct {
    int32_t op_seq_index;
    int32_t num_next_ops;
    int32_t num_dependencies;
    int32_t next_primitive_index[8];
    int32_t device_type;   /* 0 host, 1 device */
    int32_t channel;
    uint64_t params[4];
} pccl_primitive_meta;

/* One fused step: layout of the reference's FusedStep (include/engine/fused_step.h:7-22). */
typedef struct {
    int8_t primitive_type;
    int8_t pad_[3];
    int32_t peer_rank;
    int32_t offset_0;
    int32_t offset_1;
    int32_t offset_2;
    int32_t size;
    int32_t notify_signal_id;
    int32_t notify_peer_rank;
    int32_t wait_signal_id;
    int32_t wait_peer_rank;
    uint8_t has_notify;
    uint8_t has_wait;
    uint8_t pad2_[2];
} pccl_fused_step;

/* ------------------------------------------------------------------------------------------
 * Host-only graph tools (no GPU needed).
 * ------------------------------------------------------------------------------------------ */
typedef struct pccl_graph pccl_graph;
typedef struct pccl_program pccl_program;

/* Load one rank's JSON v2 graph.  Replaces GraphBuilder::loadFromFile + SmChannel/TmaChannel::parse
 * (reference csrc/engine/graph_builder.cc:12-107; csrc/plugins/cuda/channels/sm_channel.h:26-96,
 * tma_channel.h:27-81).  Missing file / no "operations" / an op without index|executor|primitive
 * -> PCCL_ERR_NOT_FOUND / PCCL_ERR_PARSE (the reference returns false); unknown primitive or
 * dtype -> PCCL_ERR_PARSE (the reference throws). */
int pccl_graph_load_file(const char* path, pccl_graph** out);
int pccl_graph_load_json(const char* text, size_t len, pccl_graph** out);
/* Build a graph from arrays an engine has already parsed (reference GraphBuilder's operators_ /
 * metadata_ vectors, include/engine/graph_builder.h).  dtype is taken from the primitive ids. */
int pccl_graph_from_triggers(const pccl_trigger* triggers, const pccl_primitive_meta* meta, int n,
                             const char* collective_type, pccl_graph** out);
void pccl_graph_free(pccl_graph* g);
int pccl_graph_num_ops(const pccl_graph* g);
int pccl_graph_dtype(const pccl_graph* g);            /* pccl_dtype of tensor_info.dtype */
int64_t pccl_graph_tensor_elems(const pccl_graph* g); /* product of tensor_info.shape, 0 if absent */
const char* pccl_graph_collective_type(const pccl_graph* g);
int pccl_graph_get_triggers(const pccl_graph* g, pccl_trigger* out, int cap);
int pccl_graph_get_meta(const pccl_graph* g, pccl_primitive_meta* out, int cap);
/* Collapse per-channel linear chains into fused steps.  Replaces GraphBuilder::buildFusedDescriptor
 * (reference csrc/engine/graph_builder.cc:163-316).  Returns the number of steps, or
 * PCCL_ERR_UNSUPPORTED when the reference would fall back to its dependency-counter runner
 * (an op with >1 dependency or successor, a chain starting with a data op, >128 steps).
 * channel_offsets must hold PCCL_HIP_MAX_CHANNELS+1 ints. */
int pccl_graph_fused_steps(const pccl_graph* g, pccl_fused_step* steps, int cap,
                           int* channel_offsets, int* num_channels);

/* What the linker derived from R per-rank graphs. */
typedef struct {
    int32_t num_vranks;
    int32_t dtype;
    int32_t num_ops;            /* all primitives over all ranks */
    int32_t num_data_ops;
    int32_t num_levels;         /* longest dependency chain over data ops */
    int32_t position_aligned;   /* 1 if every data op reads and writes the same element positions */
    int32_t num_segments;       /* column plan: maximal position ranges with one op list */
    int32_t residual_signals;   /* semaphores one execution leaves at another count than it found (0 for balanced graphs) */
    int64_t buffer_elems;       /* rank-buffer elements the graphs address (max offset+size) */
    int64_t algorithmic_bytes;  /* sum over data ops: reduce 3*n*esize, copy 2*n*esize */
    int64_t column_load_bytes;  /* bytes the column plan loads / stores from memory per execution */
    int64_t column_store_bytes;
    int32_t num_items;          /* stepwise plan: (op, tile) work items */
    int32_t num_gather_copies;  /* alltoall graphs: direct input-to-output copies the staged call composes
                                   into (0 = no such plan, the call stages through the rank buffers) */
    int64_t staged_load_bytes;  /* the same for a staged call that runs on the caller's tensors */
    int64_t staged_store_bytes; /* (0 when the graph has no such plan and staging copies are used) */
    int32_t race_checked;       /* 1: every pair of conflicting accesses was checked for an ordering; 0: the
                                   check was switched off or the program is too large for it */
    int32_t order_checked;      /* 1: the pairing of notifies and waits was checked for ambiguity; 0: the
                                   program has too many ops for the check (the pairing of one valid execution
                                   order is then used unverified) */
    int32_t chain_segments;     /* segments of the column plan in chain form (one accumulator takes every rank's
                                   original value in turn, the result goes to a set of ranks); equal to num_segments
                                   when the whole plan can run on the phased runner, else 0 */
    int32_t staged_chain_segments; /* the same for the plan of a staged call on the caller's tensors */
} pccl_program_info;

/* One data op of the linked program, for inspection and tests. */
typedef struct {
    int32_t rank, channel, op_index, is_reduce, redop, peer_rank, level, num_deps;
    int64_t offset_0, offset_1, offset_2, size;
    int32_t deps[8];            /* indices into the linked op array (first 8) */
} pccl_linked_op;

/* Link R graphs (index = rank) into one program: pair the k-th notify arriving at (target, id) with
 * the k-th wait on it (counting semaphores, reference cuda_executor.cu:414-445), derive data
 * dependencies, detect deadlock and unordered conflicting accesses.  No reference counterpart:
 * the reference runs one process per rank and synchronises at run time. */
int pccl_program_link(const pccl_graph* const* graphs, int num_vranks, pccl_program** out);
/* The same for an execution that finds semaphores above zero: `carried` holds num_carried triples
 * (rank, signal id, count), the state earlier executions left in the engine's signal region (the
 * reference zeroes it only in Engine::resetSignals, csrc/engine_c.cc:576-593).  The first `count`
 * waits on such a semaphore pass without a notify of this execution (cuda_executor.cu:425-445) and
 * are ordered after none.  An engine does this by itself (pccl_hip_execute*); this entry point is for
 * inspection and tests. */
int pccl_program_link_carried(const pccl_graph* const* graphs, int num_vranks, const int32_t* carried, int num_carried,
                              pccl_program** out);
/* The semaphores a program touches: quadruples (rank, signal id, notifies, waits) of one execution,
 * ordered by (rank, id); returns their number (fills at most `cap`).  One execution changes the count
 * of each by notifies - waits. */
int pccl_program_get_signals(const pccl_program* p, int32_t* out, int cap);
void pccl_program_free(pccl_program* p);
int pccl_program_get_info(const pccl_program* p, pccl_program_info* out);
int pccl_program_get_ops(const pccl_program* p, pccl_linked_op* out, int cap);

/* One segment of the column plan, for inspection and tests: the element positions [start, end) share
 * one column program, instruction words [prog_start, prog_start + prog_len) and first-touch list
 * words [pre_start, pre_start + pre_words) of the arrays pccl_program_get_column returns.  An
 * instruction word holds, from the low byte up: self rank, peer rank, source of a (1 memory,
 * 2 accumulator), source of b (0 none = copy, 1 memory, 2 accumulator), reduce operator, store (low
 * two bits: 0 dead, 1 read back later, 2 final; bit 2: last write of that rank), a is a first
 * touch, b is a first touch.  A first-touch word lists 8 ranks, one per byte, 0xFF = none.
 * bcast_mask: ranks that receive the accumulator after the last instruction.  The windows say which
 * positions of rank r a staged call reads from its input tensor and hands back in its output. */
typedef struct {
    int64_t start, end;
    int32_t prog_start, prog_len;
    int32_t pre_start, pre_words;
    uint64_t bcast_mask;
} pccl_column_segment;

/* which = 0: the in-place plan; 1: the plan of a staged call that runs on the caller's tensors
 * (no segments when the graph has none).  Each array is filled up to its capacity; the three
 * counts needed are returned through n_segs / n_instrs / n_pre.  in_window / out_window (which = 1,
 * may be NULL) receive 2 * num_vranks values: start and end per rank.  No reference counterpart. */
int pccl_program_get_column(const pccl_program* p, int which,
                            pccl_column_segment* segs, int seg_cap, int* n_segs,
                            uint64_t* instrs, int instr_cap, int* n_instrs,
                            uint64_t* pre, int pre_cap, int* n_pre,
                            int64_t* in_window, int64_t* out_window);

/* ------------------------------------------------------------------------------------------
 * Device executor.
 * ------------------------------------------------------------------------------------------ */
typedef struct pccl_hip_ctx pccl_hip_ctx;

/* Engine construction: replaces Engine::Engine() + BufferManager + MemoryLayout::initialize
 * (reference csrc/engine_c.cc:82-164, csrc/engine/memory_layout.cc:8-138).  Rank buffers are
 * sized on demand from the registered graphs instead of one fixed 1 GiB buffer. */
int pccl_hip_create(pccl_hip_ctx** out, int device, int num_vranks);
int pccl_hip_destroy(pccl_hip_ctx* ctx);

/* Engine::regOp(name, filename) for one virtual rank (reference csrc/engine_c.cc:166-201). */
int pccl_hip_register_file(pccl_hip_ctx* ctx, const char* name, int vrank, const char* path);
int pccl_hip_register_json(pccl_hip_ctx* ctx, const char* name, int vrank, const char* text, size_t len);
int pccl_hip_register_triggers(pccl_hip_ctx* ctx, const char* name, int vrank,
                               const pccl_trigger* triggers, const pccl_primitive_meta* meta, int n,
                               const char* collective_type);

/* Options, the counterpart of the reference's environment switches (csrc/plugins/cuda/cuda_device.cc:
 * 289-298, csrc/engine_c.cc:351): key "mode" = "auto" | "column" | "stepwise" | "persistent";
 * "num_blocks" = workgroup cap of a launch (0 = sized to the device); "check_races" = "0" | "1";
 * "timing" = "0" | "1" (record HIP events around the program); "vecs_per_thread" = 1 | 2 | 4;
 * "step_tile_bytes" (work item of the level and persistent runners: 0 = chosen from the program's
 * size, 4 to 32 KiB, else a multiple of 4096); "wait_timeout_ms" (how long a persistent launch waits
 * for a predecessor); "test_host_epoch_limit" / "test_graph_epoch_limit" (for tests: the launch number
 * at which the persistent runner's flags are cleared and its numbering restarts, on the host and for
 * launches recorded into a graph; by default about 2^30 launches apart);
 * "fuse_staging" = "1" | "0" (allreduce-type calls in column mode read the input tensors and write
 * the output tensors directly instead of staging through the engine's rank buffers);
 * "lds_slots" = "1" | "0" (column runner keeps values it re-reads in per-thread LDS slots, so each
 * rank buffer is read and written at most once per position; "0" re-reads them through memory);
 * "slot_threads" = 0 | 64 | 128 | 256 | 512 | 1024 (workgroup size of that runner, 0 = from the rank count
 * and the plan's traffic);
 * "slot_vecs" = 0 | 1 | 2 | 4 (16-byte vectors per thread of that runner: a workgroup's tile is
 * slot_threads x slot_vecs vectors of every rank; 0 = from the rank count); "slot_lds_kib" = 0..160
 * (least LDS a workgroup of that runner asks for, which bounds the workgroups per CU; 0 = chosen);
 * "slot_direct" = "1" | "0" (first touches loaded straight into LDS, or through registers);
 * "slot_store_waves" = "-1" | "0" | "1" (1: the final broadcast of a program goes through LDS and each
 * wave stores whole tiles of some ranks; 0: every wave stores a slice of every rank; -1, the default:
 * 1 for plans that write at least four times what they read, such as an allgather);
 * "phased" = "-1" | "0" | "1" (column plans in chain form - ring allreduce, staged reduce_scatter and
 * allgather, trees under an operator that may be re-associated, balanced trees of float sums - on the
 * phased runner: one persistent workgroup per CU, the whole chip reads, meets, writes, meets; -1, the
 * default: when the tensors give at least every second CU a 128 KiB chunk of each rank and the plan
 * does not store more than twice what it loads, which leaves an allgather on the slot runner);
 * "phased_shape" = "-1" | "0" | "1" (its workgroup: 512 threads x 16 vectors, or 256 x 32; -1: by rank
 * count); "phased_exchange" = "-1" | "0" | "1" (the 256 x 32 shape on chains: 1, and -1, read as slabs
 * and write with each wave on 32 KiB in a row, the sums changing hands through LDS in between; 0: each
 * wave on 32 KiB in a row for reads as well); "phased_sweeps" = "-1" | "1" | "2" (sweeps the 512 x 16
 * shape reads before it writes their sums: two make the phases longer and the meetings fewer; -1: two
 * from two sweeps on for plans on up to 8 ranks and for plans that load four times what they store,
 * which run without meetings below that); "phased_linear" = "-1" | "0" | "1" (the 256 x 32 shape with
 * the chunks of 128 neighbouring workgroups interleaved slab by slab, so that the chip sweeps each rank
 * buffer as one stream; possible on up to 8 ranks when every segment of the plan is a whole multiple of
 * 128 chunks - 16 MiB of every rank - and 128 divides the grid; also for segments of 64 chunks - of 32
 * for plans that mostly write - that lie one after the other and have the same sources count, operator
 * and store mask, a group then spanning several of them; -1: wherever possible except for plans
 * that load four times what they store; 1: for those as well); "phased_barriers" = "1" | "0" (0: no
 * meetings, for comparison); "phased_timeout_us" (how long a workgroup waits at a meeting before the
 * launch goes on unsynchronised: meetings order nothing; the environment variable PCCL_PHASED sets
 * "phased" for new contexts);
 * "level_graph" = "0" | "1" (the level runner launches level by level, or replays the launches of an
 * execution as one HIP graph captured per set of rank pointers);
 * "trace_ranges" = "0" | "1" (host-side roctx ranges around the stages of a call, under the names of
 * the reference's NVTX ranges, include/common/nvtx.h:7-16, csrc/engine_c.cc:468-489,
 * csrc/plugins/cuda/cuda_device.cc:313-319: "d2d_input_copy", "execute", "d2d_output_copy", and
 * inside "execute" "fused_kernel" for the column runner or "executor_kernel" for the level and
 * persistent runners; the marker library is loaded at run time and PCCL_ERR_UNSUPPORTED is returned
 * if there is none; the environment variable PCCL_TRACE_RANGES=1 sets it for new contexts).
 * Every value except "mode" is a whole number written as text; anything else ("on", "4k"), a value out
 * of the option's range and an unknown key return PCCL_ERR_INVALID and leave the option as it was. */
int pccl_hip_set_option(pccl_hip_ctx* ctx, const char* key, const char* value);
/* The current value of an option as text (the keys of pccl_hip_set_option, "num_vranks", "signals" -
 * the semaphores that executions so far have left above zero, as "rank:id=count" joined by commas in
 * (rank, id) order, empty when there are none; PCCL_ERR_INVALID if `cap` is too small for the text -, and
 * "runner_inplace:NAME" / "runner_staged:NAME": the kernel an in-place / staged execution of operation
 * NAME would launch now - "phased_kernel", "column_slot_kernel", "column_kernel", "level_kernel",
 * "persistent_kernel", "gather_kernel", or "staging + ..." - which links the operation; and
 * "phased_shape_inplace:NAME" / "phased_shape_staged:NAME": the phased runner's shape for operation
 * NAME as "shape=N group=K [segments=S] meetings=M" (N: 0 = 512 threads x 16 vectors, 1 / 3 = 256 x 32 without / with
 * the exchange, 2 = balanced trees, 4 = two sweeps per write phase, 5 = interleaved chunks), or "none";
 * "slot_shape:NAME": the slot runner's workgroup for operation NAME as "threads x vectors", e.g.
 * "256x2", or "0x0" if its column plan does not run there - chosen from the rank count, and larger
 * for plans that store at least four times what they load): what the
 * environment switches PCCL_NUM_BLOCKS / PCCL_DISABLE_FUSED / PCCL_TRACE_RANGES left in a new context
 * can be read back here.  No counterpart in the reference. */
int pccl_hip_get_option(pccl_hip_ctx* ctx, const char* key, char* value, size_t cap);

/* Engine::exeOp / exeOpAsync (reference csrc/engine_c.cc:269-560): for every virtual rank r copy
 * inputs[r] into rank buffer r (allgather: at r*in_bytes), run the program, copy the result to
 * outputs[r] (allreduce/default: buffer[0..out_bytes); reduce_scatter: chunk r; alltoall: own chunk
 * + scratch region).  All work is enqueued on `stream` (a hipStream_t, NULL = default stream);
 * sync != 0 waits for it. */
int pccl_hip_execute(pccl_hip_ctx* ctx, const char* name, const void* const* inputs,
                     void* const* outputs, size_t in_bytes, size_t out_bytes, void* stream, int sync);
/* Zero-copy variant: bufs[r] IS rank buffer r (every one at least buf_bytes long); no staging.
 * Buffers that are not 16-byte aligned are run by the level runner instead of the column runner.
 * No counterpart in the reference, whose rank buffers belong to the engine. */
int pccl_hip_execute_inplace(pccl_hip_ctx* ctx, const char* name, void* const* bufs, size_t buf_bytes,
                             void* stream, int sync);
/* pccl_hip_execute_inplace for callers that cannot allocate: code whose stream is being captured into a
 * graph, tight serving loops, harnesses that forbid hipMalloc.  It has no counterpart in the reference.
 * The call allocates no device memory and copies nothing: it runs the operation as ONE launch of the
 * persistent (flag-ordered) runner whose tables and progress block (error words, one flag per work
 * item, one ready word per data op, the op and dependency tables, the item-to-op map) live in a
 * workspace of PCCL_HIP_STATIC_WORKSPACE_BYTES that is part of the library's device image; what has to
 * reach the device travels in kernel arguments.  An operation that needs more (the error says how much;
 * larger work items - option "step_tile_bytes" - need less) is refused with PCCL_ERR_INVALID, and so are
 * rank buffers smaller than the graph addresses.  The first call for an operation links it on the host
 * (host memory only; pccl_hip_op_info does the same ahead of time).  Every GPU has one such workspace,
 * shared by all contexts and operations and keeping the last call's contents: when another operation
 * used it last, this call first clears the progress block and rewrites the tables (by kernels on
 * `stream`), which it refuses to do on a capturing stream (execute once outside the capture first).
 * Calls that overlap in time on one GPU - two streams, two threads - race on the workspace.
 * A recorded launch stays valid while the workspace holds its operation's tables.  Replayed after
 * another operation has taken the workspace over it executes nothing and leaves its rank buffers
 * exactly as they were (the kernel compares a tag in its arguments with the one in the workspace
 * before it reads any table).  The library notices at the next look at the workspace (a synchronous
 * call of this entry point, or pccl_hip_sync): it logs a warning that names the operation, and the
 * next pccl_hip_sync of THAT operation returns PCCL_ERR_INVALID saying so.  The call that happens to
 * notice is not failed for it: a call of this entry point that returns 0 has executed and updated its
 * buffers, one that returns PCCL_ERR_HIP for an expired wait has updated them partially, and every
 * other error is returned before anything is enqueued.  Execute the operation once more through this
 * entry point and its recorded launch works again. */
int pccl_hip_execute_inplace_static(pccl_hip_ctx* ctx, const char* name, void* const* bufs, size_t buf_bytes,
                                    void* stream, int sync);
/* Engine::syncOp (reference csrc/engine_c.cc:562-574). */
int pccl_hip_sync(pccl_hip_ctx* ctx, const char* name);
/* Engine::resetSignals (reference csrc/engine_c.cc:576-593): zero the engine's counting semaphores.
 * As in the reference they are one state per engine, shared by all registered operations, and live
 * from one execution to the next: a notify that no wait consumed is found by the next execution, of
 * any operation, that waits on that semaphore (a wait passes on a count above zero and takes one,
 * cuda_executor.cu:425-445).  This library resolves notifies and waits when it links an operation, so
 * it keeps the counts on the host (updated when an execution is issued; the caller orders executions
 * by the streams it issues them to), links an operation for the counts it finds, and links it again
 * when a later execution finds others (an operation whose notifies and waits balance, on semaphores
 * nobody left counts on - every schedule template - is linked once).  What follows from a count: a
 * wait with no notify of its own execution passes once per count and deadlocks (PCCL_ERR_LINK, before
 * anything runs) without one; a wait that passes on a carried count is ordered after nothing, so data
 * it was meant to guard may now race (reported as a data race at link time).  An execution that would
 * move or use counts is refused on a capturing stream (PCCL_ERR_INVALID): a replay could not follow
 * them.  A name that is not registered is ignored, like in the reference. */
int pccl_hip_reset_signals(pccl_hip_ctx* ctx, const char* name);

int pccl_hip_op_info(pccl_hip_ctx* ctx, const char* name, pccl_program_info* out);
/* Duration of the most recent program launch of `name` (kernel only, HIP events on its stream). */
int pccl_hip_last_kernel_ms(pccl_hip_ctx* ctx, const char* name, float* ms);

/* The two data primitives on their own (reference executeReduce / executeCopy,
 * csrc/plugins/cuda/cuda_executor.cu:60-101 -> vector_add / vector_copy, kernel/compute.h:21-102):
 * c[i] = a[i] (+|max|min) b[i], dst[i] = src[i]; any alignment, any n. */
int pccl_hip_reduce(int dtype, int redop, const void* a, const void* b, void* c, size_t n, void* stream);
int pccl_hip_copy(int dtype, const void* src, void* dst, size_t n, void* stream);

const char* pccl_hip_last_error(void);
const char* pccl_hip_version(void);

#ifdef __cplusplus
}
#endif
#endif /* PCCL_HIP_H_ */
