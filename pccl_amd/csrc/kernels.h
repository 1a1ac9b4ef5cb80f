// Device-side structures and launch wrappers of the gfx950 kernels.
#pragma once

#include <cstdint>

#include "../../include/pccl_hip.h"

// accessors usable in kernels and in the host-only translation units
#ifdef __HIPCC__
#define PCCL_HD __host__ __device__
#else
#define PCCL_HD
#endif

namespace pccl_hip {

// Rank-buffer base pointers handed to a kernel by value (kernarg segment).  Entry r is where
// rank r's stores and non-first loads go; entry MAX+r is where a first-touch load of rank r reads
// from (the same buffer, or the caller's input tensor when staging is fused into the program).
struct RankPtrs {
    char* p[2 * PCCL_HIP_MAX_VRANKS];
};

struct DevColSegment {
    int64_t start, end;      // element positions
    int64_t first_vec;       // start / vector elems
    int64_t first_tile;      // prefix sum of tiles
    int32_t prog_start, prog_len;
    int32_t pre_start, pre_words;   // first-touch rank list, 8 ranks per 64-bit word (0xFF = none)
    int32_t streaming;       // 1: every load is a first touch and every live store is final
    int32_t pad_;
    uint64_t bcast_mask;     // ranks that receive the accumulator after the last instruction
    uint64_t pre_mask;       // ranks the program reads by first touch (the pre list as a set)
};

struct DevStepOp {    // 64 bytes: one 16-dword scalar load
    int64_t off0, off1, off2, size;  // elements
    uint32_t who;    // self rank | peer rank << 8 | is_reduce << 16 | reduce operator << 24
    int32_t first_item, ntiles, dep_start, ndeps;
    int32_t lead;    // the op's items sit on a grid of tile_elems anchored `lead` elements in front of its
                     // first element, chosen so that item boundaries fall on multiples of the tile size
                     // in the destination buffer: only the first and last item of an op are ragged
    int32_t pad_[2];
    PCCL_HD int self() const { return who & 0xFF; }
    PCCL_HD int peer() const { return (who >> 8) & 0xFF; }
    PCCL_HD bool is_reduce() const { return (who >> 16) & 1; }
    PCCL_HD int redop() const { return who >> 24; }
};
static_assert(sizeof(DevStepOp) == 64, "DevStepOp is read with one scalar load");

struct StepState {      // device memory of the persistent runner
    uint32_t owner;        // shared (static) block: tag of the operation whose tables follow; 0 for an operation's own block
    int32_t graph_epoch;   // launch number of the last launch recorded into a graph (see StepwiseLaunch::epoch)
    int32_t error_op;   // 1 + index of the op whose bounded wait expired (0 = none); host clears it
    int32_t error_dep;  // 1 + index of the predecessor it was waiting for
    uint32_t stale_owner;  // tag of a launch that found another operation's tables in a shared block and did nothing
    int32_t pad[27];
    // followed by int32 flag[num_items] (the epoch of the launch that last completed the item) and
    // int32 ready[num_ops] (the epoch of the launch in which the op's first tile last saw all predecessors done)
};

struct ColumnLaunch {
    const DevColSegment* segs;
    int32_t num_segs;
    const uint64_t* instrs;   // ColInstr words
    const uint64_t* pre;      // first-touch rank lists of the segments
    int64_t total_tiles;
    int32_t dtype;
    int32_t vecs_per_thread;  // 1, 2 or 4 (register runner)
    int32_t num_blocks;       // 0: one workgroup per tile
    int32_t slot_threads;     // 0: register runner (re-read values go through memory);
                              // 64 ... 1024: workgroup size of the slot runner (re-read values in LDS)
    int32_t slot_vecs;        // slot runner: 16-byte vectors per thread (1, 2 or 4); a tile is slot_threads x slot_vecs vectors
    int32_t slot_lds_bytes;   // slot runner: dynamic LDS of a workgroup (>= num_ranks x slot_vecs x slot_threads x 16)
    int32_t num_ranks;        // slot runner: LDS slots per thread
    int32_t slot_direct;      // slot runner: 1 = first touches are loaded straight into LDS
    int32_t slot_store_waves; // slot runner: 1 = the broadcast tail goes through LDS and each wave stores whole tiles of some ranks
    int32_t xcd_run;          // run length of the tile-to-XCD mapping; filled in by the launcher
    int32_t seg_tiles;        // > 0: every segment has this many tiles (segment = tile / seg_tiles, fewer than 2^32 tiles); 0: search
};

// One segment of a chain plan (see ChainSegment in program.h) as the phased runner reads it.
struct DevChainSegment {
    int64_t start, end;        // element positions
    int64_t first_vec;         // start / vector elems
    int64_t first_chunk;       // prefix sum of chunks
    int32_t src_start, n_src;  // words in PhasedLaunch::srcs: the ranks whose values are combined, in order
    int32_t redop;
    int32_t tree_depth;        // 0: a chain; D > 0: a perfectly balanced tree over the 2^D ranks of srcs, left to right
    uint64_t store_mask;       // ranks that receive the result
};
static_assert(sizeof(DevChainSegment) == 56, "DevChainSegment is read 8 bytes at a time");

// Meeting point of the phased runner's workgroups (device memory, zero between launches: the last
// workgroup to leave a launch clears it).
struct PhaseSync {
    int32_t arrive;  int32_t pad0[31];   // arrivals at the current barrier
    int32_t release; int32_t pad1[31];   // number of the last barrier that everybody has reached
    int32_t broken;                      // a wait ran out of time: no more waiting in this launch
    int32_t exited;                      // workgroups that have left the launch
    int32_t pad2[30];
};

struct PhasedLaunch {
    const DevChainSegment* segs;
    int32_t num_segs;
    const int32_t* srcs;      // the segments' source ranks, one 32-bit word each
    int64_t total_chunks;
    int32_t seg_chunks;       // > 0: every segment has this many chunks; 0: search
    int32_t dtype;
    int32_t shape;            // 0: 512 threads x 16 vectors, 1: 256 threads x 32 vectors (each wave a contiguous 32 KiB),
                              // 2: 256 x 32 with the code for balanced trees as well; 3: as 1, but read as slabs and
                              // written with each wave on 32 KiB in a row (the sums change hands through LDS);
                              // 4: as 0, two sweeps read before their sums are written; 5: 256 x 32 slabs, the
                              // chunks of `group` workgroups interleaved slab by slab (phased_kernel_linear)
    int32_t num_blocks;       // 0: one workgroup per CU
    int32_t barriers;         // 1: all workgroups read together, then write together; 0: no meeting
    int32_t group;            // shape 5: workgroups whose chunks are interleaved (a power of two that divides the grid and every
                              // segment's chunk count; all chunks whole)
    int32_t group_segs;       // shape 5: 1, or the segments a group spans (2 or 4: the segments are then `group` / group_segs
                              // chunks long, adjacent in memory, with the same number of sources, operator and store mask,
                              // their source lists one after the other in `srcs`)
    PhaseSync* sync;
    uint64_t timeout_ticks;   // 100 MHz ticks a workgroup waits at a meeting point before it goes on alone
};
// Vectors of every rank one workgroup of the given shape takes per sweep.
PCCL_HD constexpr int64_t phased_chunk_vecs(int shape) { (void)shape; return 8192; }

struct StepwiseLaunch {
    const DevStepOp* ops;
    int32_t num_ops;
    const int32_t* deps;
    const int32_t* item_op;
    int32_t num_items;
    int64_t tile_elems;
    StepState* state;
    int32_t dtype;
    int32_t num_blocks;
    int32_t epoch;            // persistent runner: value a completed item's flag takes in this launch;
                              // 0: take it from StepState::graph_epoch, which the launcher advances first
    uint32_t owner_tag;       // persistent runner in a shared block: run only if StepState::owner equals this (0: no check)
    uint64_t timeout_ticks;   // persistent runner: 100 MHz ticks a workgroup may run before a wait gives up
    int32_t graph_epoch_limit;// recorded launches: where the device-side launch counter wraps (0: kGraphEpochLimit)
};

// Launch numbers of the persistent runner: the host counts 1 .. kHostEpochLimit and then clears the
// flags and starts again; recorded launches count kGraphEpochBase + 1 .. kGraphEpochLimit on the device.
constexpr int32_t kGraphEpochBase = 0x40000000;
constexpr int32_t kHostEpochLimit = kGraphEpochBase - 16;
constexpr int32_t kGraphEpochLimit = 0x7FFFFFF0;

// All return a hipError_t value as int (0 = success).
int launch_column(const ColumnLaunch& L, const RankPtrs& ptrs, void* stream);
int launch_persistent(const StepwiseLaunch& L, const RankPtrs& ptrs, void* stream);
int launch_phased(const PhasedLaunch& L, const RankPtrs& ptrs, void* stream);
// One dependency level: items [item_begin, item_end) of the work list.
int launch_level(const StepwiseLaunch& L, int item_begin, int item_end, const RankPtrs& ptrs, void* stream);
int launch_reduce(int dtype, int redop, const void* a, const void* b, void* c, size_t n, void* stream);
int launch_copy_bytes(const void* src, void* dst, size_t nbytes, void* stream);
// One launch copying `bytes` from src.p[r] + src_off[r] to dst.p[r] + dst_off[r] for r < R.
// One direct copy of a gather plan: `bytes` from src.p[src_rank] + src_off to dst.p[dst_rank] + dst_off;
// first_tile = tiles of all earlier copies (4 KiB tiles, one workgroup each).
struct DevGatherCopy { int64_t src_off, dst_off, bytes, first_tile; int32_t src_rank, dst_rank; };
// copy_tiles > 0: every copy has that many tiles (copy = tile / copy_tiles); 0: search the prefix sums.
int launch_gather(const DevGatherCopy* copies, int n, int64_t total_tiles, int copy_tiles, const RankPtrs& src, const RankPtrs& dst, void* stream);

struct StageOffsets { int64_t src[PCCL_HIP_MAX_VRANKS]; int64_t dst[PCCL_HIP_MAX_VRANKS]; };
int launch_stage(const RankPtrs& src, const RankPtrs& dst, const StageOffsets& off, int R, size_t bytes, void* stream);
int launch_fill_zero(void* dst, size_t nbytes, void* stream);

// The static workspace of `device` (which must be the current device the first time): its device
// address and size.  Returns a hipError_t value.
int static_workspace(int device, void** ptr, size_t* bytes);
// `nbytes` (a multiple of 8) of host memory to device memory at `dst` through kernel arguments.
struct TablePayload { uint64_t w[448]; };   // 3.5 KiB: a kernel's arguments may take 4 KiB
int launch_table_write(const void* src, size_t nbytes, void* dst, void* stream);
int launch_item_op_fill(const DevStepOp* ops, int num_ops, int32_t* item_op, void* stream);

int device_cu_count(int device);

}  // namespace pccl_hip
