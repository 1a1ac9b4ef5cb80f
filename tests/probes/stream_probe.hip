// Memory-system probe for two design decisions of the executor's kernels, with no tables and no
// arithmetic in the way:
//
//   width    a 1 GiB out-of-place copy in 4 KiB tiles, every lane moving 16 bytes per tile as four
//            4-byte, two 8-byte or one 16-byte access (the kernels use 16)
//   streams  what the column runner's traffic looks like: a workgroup loads one 16-byte vector per
//            thread from each of R buffers at the same offset - all loads first - and stores R
//            vectors, either back in place (an in-place execution) or to R other buffers (a staged
//            call run on the caller's tensors); 4 GiB of buffers in every case
//
//   ceilings what the memory system gives a kernel that only reads 4 GiB, only writes 4 GiB, or
//            copies 2 GiB to another 2 GiB, one 16-byte access per lane and 4 KiB tile, with plain
//            non-temporal stores and with non-temporal agent-scope (nt sc1) stores
//
// Usage: stream_probe [width|streams|ceilings|all]; prints one line per case.  Tiles are dealt to the XCDs in
// runs of 256 like the library's kernels do.
#include <hip/hip_runtime.h>

#include <cstdio>
#include <cstdlib>
#include <cstring>

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

#define CHECK(expr)                                                                         \
    do {                                                                                    \
        hipError_t e_ = (expr);                                                             \
        if (e_ != hipSuccess) { std::fprintf(stderr, "%s: %s\n", #expr, hipGetErrorString(e_)); std::exit(1); } \
    } while (0)

constexpr int kRun = 256;   // tiles per XCD in a row
constexpr int kMaxStreams = 32;
struct Ptrs { char* p[kMaxStreams]; };

__device__ __forceinline__ int64_t xcd_tile(int64_t w) {
    const int64_t in = w & ((int64_t)8 * kRun - 1);
    return w - in + ((in & 7) * kRun) + (in >> 3);
}

// W = bytes per access.  A tile is 4 KiB; lane t moves bytes [16 t, 16 t + 16) of every 4 KiB tile
// when W = 16, and accesses number i of a lane are W x 256 bytes apart otherwise, so that every
// single access of a wave is contiguous.
template <int W>
__global__ __launch_bounds__(256) void copy_width(const char* src, char* dst, int64_t tiles) {
    const int64_t tile = xcd_tile(blockIdx.x);
    if (tile >= tiles) return;
    const char* s = src + tile * 4096;
    char* d = dst + tile * 4096;
    const int t = threadIdx.x;
    if constexpr (W == 16) {
        __builtin_nontemporal_store(__builtin_nontemporal_load((const u32x4*)s + t), (u32x4*)d + t);
    } else if constexpr (W == 8) {
        u32x2 v[2];
#pragma unroll
        for (int i = 0; i < 2; ++i) v[i] = __builtin_nontemporal_load((const u32x2*)s + i * 256 + t);
#pragma unroll
        for (int i = 0; i < 2; ++i) __builtin_nontemporal_store(v[i], (u32x2*)d + i * 256 + t);
    } else {
        uint32_t v[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) v[i] = __builtin_nontemporal_load((const uint32_t*)s + i * 256 + t);
#pragma unroll
        for (int i = 0; i < 4; ++i) __builtin_nontemporal_store(v[i], (uint32_t*)d + i * 256 + t);
    }
}

template <int R>
__global__ __launch_bounds__(256) void touch(Ptrs in, Ptrs out, int64_t tiles) {
    const int64_t tile = xcd_tile(blockIdx.x);
    if (tile >= tiles) return;
    const int64_t off = (tile * 256 + threadIdx.x) * 16;
    u32x4 v[R];
#pragma unroll
    for (int r = 0; r < R; ++r) v[r] = __builtin_nontemporal_load((const u32x4*)(in.p[r] + off));
#pragma unroll
    for (int r = 0; r < R; ++r) { v[r].x += 1; __builtin_nontemporal_store(v[r], (u32x4*)(out.p[r] + off)); }
}

// MODE 0: read only (the sum of what a lane read is stored only if it equals a value it cannot
// have, so that the loads stay); 1: write only; 2: copy.  SC1: stores as raw buffer stores marked
// nt sc1 (wave-uniform base, 32-bit lane offset), else plain non-temporal pointer stores.
template <int MODE, bool SC1>
__global__ __launch_bounds__(256) void ceiling(const char* src, char* dst, int64_t tiles, uint32_t never) {
    const int64_t tile = xcd_tile(blockIdx.x);
    if (tile >= tiles) return;
    const int lane_off = threadIdx.x * 16;
    u32x4 v = u32x4{1, 2, 3, 4};
    if constexpr (MODE != 1) v = __builtin_nontemporal_load((const u32x4*)(src + tile * 4096 + lane_off));
    if constexpr (MODE == 0) {
        if ((v.x ^ v.y ^ v.z ^ v.w) != never) return;
    }
    char* d = dst + tile * 4096;
    if constexpr (SC1) {
        __builtin_amdgcn_raw_buffer_store_b128(v, __builtin_amdgcn_make_buffer_rsrc((void*)d, 0, 0x7FFFFFFF, 0x00020000), lane_off, 0, 16 | 2);
    } else {
        __builtin_nontemporal_store(v, (u32x4*)(d + lane_off));
    }
}

static unsigned grid_for(int64_t tiles) {
    const int64_t span = (int64_t)8 * kRun;
    return (unsigned)((tiles + span - 1) / span * span);
}

template <class Launch>
static float timed_ms(Launch&& launch, int reps) {
    hipEvent_t e0, e1;
    CHECK(hipEventCreate(&e0));
    CHECK(hipEventCreate(&e1));
    for (int i = 0; i < 3; ++i) launch();
    CHECK(hipEventRecord(e0, 0));
    for (int i = 0; i < reps; ++i) launch();
    CHECK(hipEventRecord(e1, 0));
    CHECK(hipEventSynchronize(e1));
    float ms = 0;
    CHECK(hipEventElapsedTime(&ms, e0, e1));
    CHECK(hipEventDestroy(e0));
    CHECK(hipEventDestroy(e1));
    return ms / reps;
}

template <int W>
static void width_case(const char* src, char* dst, size_t bytes) {
    const int64_t tiles = (int64_t)(bytes / 4096);
    const float ms = timed_ms([&] { hipLaunchKernelGGL(copy_width<W>, dim3(grid_for(tiles)), dim3(256), 0, 0, src, dst, tiles); }, 20);
    std::printf("width   copy of %zu MiB, %2d bytes per access: %.4f ms, %.0f GB/s (read + write)\n", bytes >> 20, W, ms, 2.0 * bytes / ms / 1e6);
    std::fflush(stdout);
}

template <int R>
static void streams_case(bool in_place) {
    const size_t total = (size_t)4 << 30;   // bytes read (and as many written) per launch
    const size_t per = total / R;
    Ptrs in{}, out{};
    for (int r = 0; r < R; ++r) {
        CHECK(hipMalloc((void**)&in.p[r], per));
        CHECK(hipMemset(in.p[r], 0, per));
        if (in_place) out.p[r] = in.p[r];
        else { CHECK(hipMalloc((void**)&out.p[r], per)); CHECK(hipMemset(out.p[r], 0, per)); }
    }
    const int64_t tiles = (int64_t)(per / 4096);
    const float ms = timed_ms([&] { hipLaunchKernelGGL(touch<R>, dim3(grid_for(tiles)), dim3(256), 0, 0, in, out, tiles); }, 10);
    std::printf("streams R=%2d buffers of %4zu MiB, %s: %.4f ms, %.0f GB/s (read + write)\n", R, per >> 20,
                in_place ? "stored back in place " : "stored to R other ones", ms, 2.0 * total / ms / 1e6);
    std::fflush(stdout);
    for (int r = 0; r < R; ++r) {
        CHECK(hipFree(in.p[r]));
        if (!in_place) CHECK(hipFree(out.p[r]));
    }
}

template <int MODE, bool SC1>
static void ceiling_case(const char* src, char* dst, size_t bytes, const char* label) {
    const int64_t tiles = (int64_t)(bytes / 4096);
    // the buffers hold zeros, so the exclusive-or of a lane's four words is never 0xDEADBEEF
    const float ms = timed_ms([&] { hipLaunchKernelGGL((ceiling<MODE, SC1>), dim3(grid_for(tiles)), dim3(256), 0, 0, src, dst, tiles, 0xDEADBEEFu); }, 10);
    const double moved = MODE == 2 ? 2.0 * bytes : 1.0 * bytes;
    std::printf("ceiling %-34s %.4f ms, %.0f GB/s\n", label, ms, moved / ms / 1e6);
    std::fflush(stdout);
}

int main(int argc, char** argv) {
    const char* what = argc > 1 ? argv[1] : "all";
    const bool all = std::strcmp(what, "all") == 0;
    if (all || std::strcmp(what, "width") == 0) {
        const size_t bytes = (size_t)1 << 30;
        char *src = nullptr, *dst = nullptr;
        CHECK(hipMalloc((void**)&src, bytes));
        CHECK(hipMalloc((void**)&dst, bytes));
        CHECK(hipMemset(src, 1, bytes));
        CHECK(hipMemset(dst, 0, bytes));
        width_case<4>(src, dst, bytes);
        width_case<8>(src, dst, bytes);
        width_case<16>(src, dst, bytes);
        CHECK(hipFree(src));
        CHECK(hipFree(dst));
    }
    if (all || std::strcmp(what, "streams") == 0) {
        for (int in_place = 1; in_place >= 0; --in_place) {
            streams_case<1>(in_place);
            streams_case<2>(in_place);
            streams_case<4>(in_place);
            streams_case<8>(in_place);
            streams_case<16>(in_place);
            streams_case<32>(in_place);
        }
    }
    if (all || std::strcmp(what, "ceilings") == 0) {
        const size_t bytes = (size_t)4 << 30;
        char *a = nullptr, *b = nullptr;
        CHECK(hipMalloc((void**)&a, bytes));
        CHECK(hipMalloc((void**)&b, bytes));
        CHECK(hipMemset(a, 0, bytes));
        CHECK(hipMemset(b, 0, bytes));
        ceiling_case<0, false>(a, b, bytes, "read 4 GiB:");
        ceiling_case<1, false>(a, b, bytes, "write 4 GiB, nt stores:");
        ceiling_case<1, true>(a, b, bytes, "write 4 GiB, nt sc1 stores:");
        ceiling_case<2, false>(a, b, bytes / 2, "copy 2 GiB, nt stores:");
        ceiling_case<2, true>(a, b, bytes / 2, "copy 2 GiB, nt sc1 stores:");
        CHECK(hipFree(a));
        CHECK(hipFree(b));
    }
    CHECK(hipDeviceSynchronize());
    return 0;
}
