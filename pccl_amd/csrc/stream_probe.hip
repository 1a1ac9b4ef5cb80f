// Memory-system probe for the column and phased runners: bare kernels of their traffic shapes
// (R rank buffers summed position by position with integer adds, the sum stored to all R in place),
// hard-coded, with no tables and no instruction words, so that what the runners achieve can be set
// against what the GPU gives a kernel of that shape.  Standalone (HIP runtime only, not linked into
// the library); built by pccl_amd/build.py, run through `bench.py --probe "<arguments>"`.
//
//   stream_probe <ranks> <bytes per rank> <case> [<case> ...]
//   case = tile:T:V:S:W      one tile of T x V vectors per workgroup, first touches through a ring of S
//                            LDS slots per thread (S >= ranks: all in flight at once, the slot runner's
//                            shape); W = 1: the final stores dealt to the waves
//          phased:T:V:S:M:L  one persistent workgroup per CU, sums of T x V vectors in registers, ring
//                            of S slots; M = 0 no meetings, 1 all workgroups meet after the reads and after
//                            the writes, 2 meet before the reads only; L = 1: a wave's vectors contiguous;
//                            L = 2: read as slabs, written with a wave's vectors contiguous (the sums
//                            change hands through LDS between the phases)
//                            L = 3 / 4 / 5: slabs, the chunks of 128 / 256 / 64 neighbouring workgroups interleaved
//                            slab by slab - at every step the group reads or writes one contiguous piece of a rank
//          sweeps:K:A        the 512 x 16 phased shape (ring of 4, meetings) reading K sweeps - K chunks
//                            of every rank, one after the other - before their sums are written; A = 1:
//                            the sums go to every rank (an allreduce in place), A = 0: to one rank per
//                            chunk (the traffic of a reduce_scatter); K = 0: one sweep, no meetings
//          read:T / write:T / copy:T   streams only: every workgroup of T threads reads (writes) one
//                            1 KiB-per-wave tile of every rank; copy: rank r to rank (r + ranks / 2)
// Every case prints one JSON line; results are checked on the host for the cases that compute.
#include <hip/hip_runtime.h>

#include <algorithm>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <string>
#include <vector>

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
#define G1 __attribute__((address_space(1)))
#define L3 __attribute__((address_space(3)))
#define CHECK(expr) do { hipError_t e_ = (expr); if (e_ != hipSuccess) { std::fprintf(stderr, "%s: %s\n", #expr, hipGetErrorString(e_)); std::exit(1); } } while (0)

constexpr int kMaxR = 64;
struct Ptrs { char* p[kMaxR]; };
struct Meet { int arrive; int pad0[31]; int release; int pad1[31]; int failed; int pad2[31]; unsigned long long stamps[3 * 64]; };

__device__ __forceinline__ int64_t xcd_tile(int64_t w, int run_shift) {   // tiles dealt to the 8 XCDs in runs
    const int64_t span = (int64_t)8 << run_shift;
    const int64_t in = w & (span - 1);
    return w - in + ((in & 7) << run_shift) + (in >> 3);
}
__device__ __forceinline__ void st_stream(char* p, u32x4 v) {
    asm volatile("global_store_dwordx4 %0, %1, off sc1 nt\n\ts_nop 0" : : "v"((G1 u32x4*)p), "v"(v) : "memory");
}
__device__ __forceinline__ u32x4 ld_stream(const char* p) { return __builtin_nontemporal_load((const G1 u32x4*)p); }
__device__ __forceinline__ void lds_direct(const char* g, u32x4* wave_base) {
    __builtin_amdgcn_global_load_lds((const G1 void*)g, (L3 void*)wave_base, 16, 0, 2);
}
__device__ __forceinline__ void wait_vm(int n) {
    switch (n) {
#define C(i) case i: asm volatile("s_waitcnt vmcnt(" #i ")" ::: "memory"); break;
        C(0) C(1) C(2) C(3) C(4) C(5) C(6) C(7) C(8) C(9) C(10) C(11) C(12) C(13) C(14) C(15)
        C(16) C(17) C(18) C(19) C(20) C(21) C(22) C(23) C(24) C(25) C(26) C(27) C(28) C(29) C(30) C(31)
#undef C
        default: asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); break;   // conservative beyond the table
    }
}

// ---- one tile per workgroup --------------------------------------------------------------------
template <int V>
__global__ __launch_bounds__(1024 / V) void tile_kernel(Ptrs p, int R, int S, int64_t tiles, int run_shift, int wave_stores) {
    extern __shared__ u32x4 lds[];
    const int T = blockDim.x, tid = threadIdx.x;
    const int64_t tile = xcd_tile(blockIdx.x, run_shift);
    if (tile >= tiles) return;
    const int64_t vbase = tile * T * V;
    int64_t off[V];
#pragma unroll
    for (int v = 0; v < V; ++v) off[v] = (vbase + v * T + tid) * 16;
    const int first = S < R ? S : R;
    for (int r = 0; r < first; ++r)
#pragma unroll
        for (int v = 0; v < V; ++v) lds_direct(p.p[r] + off[v], lds + (r * V + v) * T + (tid & ~63));
    u32x4 acc[V];
#pragma unroll
    for (int v = 0; v < V; ++v) acc[v] = u32x4{0, 0, 0, 0};
    if (S >= R) {
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        for (int r = 0; r < R; ++r)
#pragma unroll
            for (int v = 0; v < V; ++v) acc[v] += lds[(r * V + v) * T + tid];
    } else {
        int slot = 0;
        for (int r = 0; r < R; ++r) {
            const int issued = r + S < R ? r + S : R;
            wait_vm((issued - r - 1) * V);
#pragma unroll
            for (int v = 0; v < V; ++v) acc[v] += lds[(slot * V + v) * T + tid];
            if (r + S < R) {
                asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
#pragma unroll
                for (int v = 0; v < V; ++v) lds_direct(p.p[r + S] + off[v], lds + (slot * V + v) * T + (tid & ~63));
            }
            slot = slot + 1 == S ? 0 : slot + 1;
        }
    }
    if (wave_stores) {
        __syncthreads();
#pragma unroll
        for (int v = 0; v < V; ++v) lds[v * T + tid] = acc[v];
        __syncthreads();
        const int W = T >> 6, w = tid >> 6, lane = tid & 63;
        for (int r = w; r < R; r += W) {
            char* dst = p.p[r] + vbase * 16;
            for (int j = 0; j < T * V; j += 64) st_stream(dst + (int64_t)(j + lane) * 16, lds[j + lane]);
        }
    } else {
        for (int r = 0; r < R; ++r)
#pragma unroll
            for (int v = 0; v < V; ++v) st_stream(p.p[r] + off[v], acc[v]);
    }
}

// ---- phased: persistent grid, reads / meeting / writes / meeting -----------------------------------
__device__ __forceinline__ void meet_arrive(Meet* s, int gen, int G) {
    if (threadIdx.x == 0) {
        const int old = __hip_atomic_fetch_add(&s->arrive, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if (old + 1 == gen * G) __hip_atomic_store(&s->release, gen, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
}
__device__ __forceinline__ void meet_wait(Meet* s, int gen) {     // bounded: 0.2 s
    if (threadIdx.x == 0) {
        const uint64_t t0 = __builtin_amdgcn_s_memrealtime();
        while (__hip_atomic_load(&s->release, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) < gen) {
            if (__builtin_amdgcn_s_memrealtime() - t0 > 20000000ull) { s->failed = 1; break; }
            __builtin_amdgcn_s_sleep(4);
        }
    }
    __syncthreads();
}

template <int T, int V, int S, int LAY>
__global__ __launch_bounds__(T) void phased_probe(Ptrs p, int R, int64_t chunks, int mode, Meet* meet) {
    extern __shared__ u32x4 lds[];
    static_assert(S <= V && V % S == 0, "ring");
    const int tid = threadIdx.x;
    const int G = gridDim.x;
    const int place = (blockIdx.x & 7) * (G >> 3) + (blockIdx.x >> 3);
    u32x4* const my = lds + (tid & ~63);
    const u32x4* const mine = lds + tid;
    int gen = 0;
    const int64_t sweeps = (chunks + G - 1) / G;
    constexpr bool WAVEC = LAY == 1;
    constexpr bool GROUPED = LAY >= 3;
    const int K = LAY == 3 ? 128 : LAY == 4 ? 256 : 64;                       // GROUPED: workgroups per group (the host checks that it divides the grid)
    const int64_t VS = GROUPED ? (int64_t)K * T * 16 : WAVEC ? 64 * 16 : (int64_t)T * 16;
    const int64_t WVS = GROUPED ? VS : LAY >= 1 ? 64 * 16 : (int64_t)T * 16;
    for (int64_t it = 0; it < sweeps; ++it) {
        const int64_t chunk = it * G + place;
        const bool live = chunk < chunks;
        // GROUPED: slab v of workgroup j of a group is piece (v K + j) of the group's K chunks
        const int64_t base = GROUPED ? (((chunk / K) * V * K + chunk % K) * T + tid) * 16
                           : WAVEC ? (chunk * V * T + (int64_t)(tid >> 6) * V * 64 + (tid & 63)) * 16 : (chunk * V * T + tid) * 16;
        const int64_t wbase = GROUPED ? base : LAY >= 1 ? (chunk * V * T + (int64_t)(tid >> 6) * V * 64 + (tid & 63)) * 16 : base;
        u32x4 acc[V];
#pragma unroll
        for (int v = 0; v < V; ++v) acc[v] = u32x4{0, 0, 0, 0};
        if (mode == 2) { asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); __syncthreads(); ++gen; meet_arrive(meet, gen, G); meet_wait(meet, gen); }
        if (blockIdx.x == 0 && tid == 0 && it < 64) meet->stamps[3 * it] = __builtin_amdgcn_s_memrealtime();
        if (live) {
#pragma unroll
            for (int q = 0; q < S; ++q) lds_direct(p.p[0] + base + (int64_t)q * VS, my + q * T);
            for (int r = 0; r < R; ++r) {
                const bool last_rank = r + 1 == R;
                const char* cur = p.p[r];
                const char* next = p.p[last_rank ? r : r + 1];
#pragma unroll
                for (int v = 0; v < V; ++v) {
                    if (last_rank && v + S >= V) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
                    else asm volatile("s_waitcnt vmcnt(%0)" :: "n"(S - 1) : "memory");
                    acc[v] += mine[(v % S) * T];
                    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
                    if (v + S < V) lds_direct(cur + base + (int64_t)(v + S) * VS, my + (v % S) * T);
                    else if (!last_rank) lds_direct(next + base + (int64_t)(v + S - V) * VS, my + (v % S) * T);
                }
            }
        }
        if (LAY == 2) {      // read as slabs, write with each wave on V KiB in a row: the sums change hands through LDS
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            __syncthreads();
#pragma unroll
            for (int v = 0; v < V; ++v) lds[v * T + tid] = acc[v];
            __syncthreads();
            const int wb = (tid >> 6) * V * 64 + (tid & 63);
#pragma unroll
            for (int v = 0; v < V; ++v) acc[v] = lds[wb + v * 64];
            if (mode != 1) __syncthreads();
        }
        if (mode == 1) { asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); __syncthreads(); ++gen; meet_arrive(meet, gen, G); meet_wait(meet, gen); }
        if (blockIdx.x == 0 && tid == 0 && it < 64) meet->stamps[3 * it + 1] = __builtin_amdgcn_s_memrealtime();
        if (live) {
            for (int r = 0; r < R; ++r) {
                char* dst = p.p[r] + wbase;
#pragma unroll
                for (int v = 0; v < V; ++v) st_stream(dst + (int64_t)v * WVS, acc[v]);
            }
        }
        if (mode == 1) { asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); __syncthreads(); ++gen; meet_arrive(meet, gen, G); meet_wait(meet, gen); }
        if (blockIdx.x == 0 && tid == 0 && it < 64) meet->stamps[3 * it + 2] = __builtin_amdgcn_s_memrealtime();
    }
}

// ---- sweeps: K sweeps read before their sums are written ---------------------------------------------
template <int KK, bool ALL, bool MEET>
__global__ __launch_bounds__(512) void sweeps_probe(Ptrs p, int R, int64_t chunks, Meet* meet) {
    constexpr int T = 512, V = 16, S = 4;
    extern __shared__ u32x4 lds[];
    const int tid = threadIdx.x;
    const int G = gridDim.x;
    const int place = (blockIdx.x & 7) * (G >> 3) + (blockIdx.x >> 3);
    u32x4* const my = lds + (tid & ~63);
    const u32x4* const mine = lds + tid;
    int gen = 0;
    const int64_t sweeps = (chunks + G - 1) / G;
    constexpr int64_t VS = (int64_t)T * 16;
    for (int64_t it0 = 0; it0 < sweeps; it0 += KK) {
        u32x4 acc[KK][V];
#pragma unroll
        for (int k = 0; k < KK; ++k) {
            const int64_t chunk = (it0 + k) * G + place;
            const int64_t base = (chunk * V * T + tid) * 16;
#pragma unroll
            for (int v = 0; v < V; ++v) acc[k][v] = u32x4{0, 0, 0, 0};
            if (it0 + k < sweeps && chunk < chunks) {
#pragma unroll
                for (int q = 0; q < S; ++q) lds_direct(p.p[0] + base + (int64_t)q * VS, my + q * T);
                for (int r = 0; r < R; ++r) {
                    const bool last_rank = r + 1 == R;
                    const char* cur = p.p[r];
                    const char* next = p.p[last_rank ? r : r + 1];
#pragma unroll
                    for (int v = 0; v < V; ++v) {
                        if (last_rank && v + S >= V) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
                        else asm volatile("s_waitcnt vmcnt(%0)" :: "n"(S - 1) : "memory");
                        acc[k][v] += mine[(v % S) * T];
                        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
                        if (v + S < V) lds_direct(cur + base + (int64_t)(v + S) * VS, my + (v % S) * T);
                        else if (!last_rank) lds_direct(next + base + (int64_t)(v + S - V) * VS, my + (v % S) * T);
                    }
                }
            }
        }
        if (MEET) { asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); __syncthreads(); ++gen; meet_arrive(meet, gen, G); meet_wait(meet, gen); }
#pragma unroll
        for (int k = 0; k < KK; ++k) {
            const int64_t chunk = (it0 + k) * G + place;
            if (it0 + k < sweeps && chunk < chunks) {
                for (int r = ALL ? 0 : (int)(chunk % R); r < (ALL ? R : (int)(chunk % R) + 1); ++r) {
                    char* dst = p.p[r] + (chunk * V * T + tid) * 16;
#pragma unroll
                    for (int v = 0; v < V; ++v) st_stream(dst + (int64_t)v * VS, acc[k][v]);
                }
            }
        }
        if (MEET) { asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); __syncthreads(); ++gen; meet_arrive(meet, gen, G); meet_wait(meet, gen); }
    }
}

// ---- streams only ----------------------------------------------------------------------------------
// kind 0: read every rank, 1: write every rank, 2: copy rank r to rank r + R / 2
__global__ __launch_bounds__(1024) void stream_kernel(Ptrs p, int R, int64_t tiles, int run_shift, int kind, u32x4* sink) {
    const int T = blockDim.x, tid = threadIdx.x;
    const int64_t tile = xcd_tile(blockIdx.x, run_shift);
    if (tile >= tiles) return;
    const int64_t off = (tile * T + tid) * 16;
    u32x4 acc = u32x4{1, 2, 3, 4};
    if (kind == 0) {
        for (int r = 0; r < R; ++r) acc += ld_stream(p.p[r] + off);
        if (acc.x == 0x12345678u && acc.y == 0x9ABCDEF0u) sink[0] = acc;     // never true for the probe's data; keeps the loads
    } else if (kind == 1) {
        for (int r = 0; r < R; ++r) st_stream(p.p[r] + off, acc);
    } else {
        for (int r = 0; r < R / 2; ++r) st_stream(p.p[r + R / 2] + off, ld_stream(p.p[r] + off));
    }
}

// ---- host ------------------------------------------------------------------------------------------
static std::vector<int> fields(const std::string& s) {
    std::vector<int> out;
    size_t a = s.find(':');
    while (a != std::string::npos) {
        const size_t b = s.find(':', a + 1);
        out.push_back(std::atoi(s.substr(a + 1, b == std::string::npos ? std::string::npos : b - a - 1).c_str()));
        a = b;
    }
    return out;
}

int main(int argc, char** argv) {
    if (argc < 4) { std::fprintf(stderr, "usage: stream_probe <ranks> <bytes per rank> <case> ...\n"); return 2; }
    const int R = std::atoi(argv[1]);
    const size_t bytes = std::strtoull(argv[2], nullptr, 10);
    if (R < 1 || R > kMaxR || bytes < (1u << 20) || bytes % (1u << 20)) { std::fprintf(stderr, "ranks 1..64, bytes a multiple of 1 MiB\n"); return 2; }
    Ptrs p{};
    for (int r = 0; r < R; ++r) CHECK(hipMalloc(&p.p[r], bytes));
    Meet* meet; CHECK(hipMalloc(&meet, sizeof(Meet)));
    u32x4* sink; CHECK(hipMalloc(&sink, 64));
    std::vector<uint32_t> host(bytes / 4);
    hipEvent_t e0, e1;
    CHECK(hipEventCreate(&e0)); CHECK(hipEventCreate(&e1));
    int cus = 256;
    CHECK(hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, 0));
    const int reps = 10;
    auto fill = [&]() { for (int r = 0; r < R; ++r) { std::fill(host.begin(), host.end(), (uint32_t)(r + 1)); CHECK(hipMemcpy(p.p[r], host.data(), bytes, hipMemcpyHostToDevice)); } };
    auto verify = [&](size_t words) {
        const uint32_t want = (uint32_t)R * (R + 1) / 2;
        for (int r = 0; r < R; r += std::max(1, R - 1)) {
            CHECK(hipMemcpy(host.data(), p.p[r], bytes, hipMemcpyDeviceToHost));
            for (size_t i = 0; i < words; ++i) if (host[i] != want) return false;
        }
        return true;
    };
    for (int a = 3; a < argc; ++a) {
        const std::string c = argv[a];
        const std::vector<int> f = fields(c);
        float total = 0, best = 1e30f;
        double moved = 0;
        bool ok = true;
        std::string extra;
        auto timed = [&](auto&& launch) {
            for (int i = 0; i < 3; ++i) launch();
            CHECK(hipDeviceSynchronize());
            for (int i = 0; i < reps; ++i) {
                CHECK(hipEventRecord(e0, 0));
                launch();
                CHECK(hipEventRecord(e1, 0));
                CHECK(hipEventSynchronize(e1));
                float ms = 0; CHECK(hipEventElapsedTime(&ms, e0, e1));
                total += ms; best = std::min(best, ms);
            }
        };
        if (c.rfind("tile:", 0) == 0 && f.size() == 4) {
            const int T = f[0], V = f[1], S = std::min(f[2], R), W = f[3];
            const size_t lds = (size_t)S * V * T * 16;
            if ((V != 1 && V != 2 && V != 4) || T * V > 1024 || T % 64 || lds > 160 * 1024 || (S < R && (S - 1) * V > 31)) { std::printf("{\"case\": \"%s\", \"error\": \"shape not available\"}\n", c.c_str()); continue; }
            const int64_t tiles = bytes / ((int64_t)T * V * 16);
            int run = 256; while (run > 1 && 8 * run > tiles) run >>= 1;
            const int64_t grid = (tiles + 8 * run - 1) / (8 * run) * (8 * run);
            auto go = [&](auto k) {
                if (lds > 64 * 1024) CHECK(hipFuncSetAttribute(reinterpret_cast<const void*>(k), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
                auto launch = [&]() { hipLaunchKernelGGL(k, dim3((unsigned)grid), dim3(T), lds, 0, p, R, S, tiles, __builtin_ctz(run), W); CHECK(hipGetLastError()); };
                fill(); launch(); CHECK(hipDeviceSynchronize());
                ok = verify((size_t)tiles * T * V * 4);
                timed(launch);
            };
            if (V == 1) go(tile_kernel<1>); else if (V == 2) go(tile_kernel<2>); else go(tile_kernel<4>);
            moved = 2.0 * R * (double)tiles * T * V * 16;
        } else if (c.rfind("phased:", 0) == 0 && f.size() == 5) {
            const int T = f[0], V = f[1], S = f[2], mode = f[3], L = f[4];
            const int64_t chunks = bytes / ((int64_t)T * V * 16);
            auto go = [&](auto k, int lds) {
                if (lds > 64 * 1024) CHECK(hipFuncSetAttribute(reinterpret_cast<const void*>(k), hipFuncAttributeMaxDynamicSharedMemorySize, lds));
                auto launch = [&]() {
                    CHECK(hipMemsetAsync(meet, 0, sizeof(Meet), 0));
                    hipLaunchKernelGGL(k, dim3(cus), dim3(T), (size_t)lds, 0, p, R, chunks, mode, meet);
                    CHECK(hipGetLastError());
                };
                fill(); launch(); CHECK(hipDeviceSynchronize());
                ok = verify((size_t)chunks * T * V * 4);
                timed(launch);
                Meet hm; CHECK(hipMemcpy(&hm, meet, sizeof(hm), hipMemcpyDeviceToHost));
                if (hm.failed) ok = false;
                const long long sw = std::min<long long>(64, (chunks + cus - 1) / cus);
                double rd = 0, wr = 0;
                for (long long i = 0; i < sw; ++i) { rd += (double)(hm.stamps[3 * i + 1] - hm.stamps[3 * i]); wr += (double)(hm.stamps[3 * i + 2] - hm.stamps[3 * i + 1]); }
                const double per_phase = (double)R * chunks * T * V * 16 / (double)((chunks + cus - 1) / cus);
                char buf[256];
                std::snprintf(buf, sizeof buf, ", \"sweeps\": %lld, \"read_phase_us\": %.2f, \"read_phase_GBps\": %.0f, \"write_phase_us\": %.2f, \"write_phase_GBps\": %.0f",
                              (long long)((chunks + cus - 1) / cus), rd / sw / 100.0, per_phase / (rd / sw / 100.0) / 1e3, wr / sw / 100.0, per_phase / (wr / sw / 100.0) / 1e3);
                extra = buf;
            };
            // the 84 KiB keep a second workgroup off the CU
            const int lds = std::max(84 * 1024, L == 2 ? T * V * 16 : S * T * 16);
            const int group = L == 3 ? 128 : L == 4 ? 256 : L == 5 ? 64 : 1;
            if (cus % group || chunks % group) { std::printf("{\"case\": \"%s\", \"error\": \"the group does not divide the grid or the chunks\"}\n", c.c_str()); continue; }
            if (T == 512 && V == 16 && S == 4 && L == 0) go(phased_probe<512, 16, 4, 0>, lds);
            else if (T == 512 && V == 16 && S == 4 && L == 1) go(phased_probe<512, 16, 4, 1>, lds);
            else if (T == 512 && V == 16 && S == 4 && L == 2) go(phased_probe<512, 16, 4, 2>, lds);
            else if (T == 512 && V == 16 && S == 8 && L == 0) go(phased_probe<512, 16, 8, 0>, lds);
            else if (T == 256 && V == 32 && S == 8 && L == 0) go(phased_probe<256, 32, 8, 0>, lds);
            else if (T == 256 && V == 32 && S == 8 && L == 1) go(phased_probe<256, 32, 8, 1>, lds);
            else if (T == 256 && V == 32 && S == 8 && L == 2) go(phased_probe<256, 32, 8, 2>, lds);
            else if (T == 256 && V == 32 && S == 8 && L == 3) go(phased_probe<256, 32, 8, 3>, lds);
            else if (T == 256 && V == 32 && S == 8 && L == 4) go(phased_probe<256, 32, 8, 4>, lds);
            else if (T == 256 && V == 32 && S == 8 && L == 5) go(phased_probe<256, 32, 8, 5>, lds);
            else if (T == 512 && V == 16 && S == 4 && L == 3) go(phased_probe<512, 16, 4, 3>, lds);
            else if (T == 512 && V == 16 && S == 4 && L == 4) go(phased_probe<512, 16, 4, 4>, lds);
            else if (T == 256 && V == 32 && S == 16 && L == 1) go(phased_probe<256, 32, 16, 1>, lds);
            else if (T == 1024 && V == 8 && S == 8 && L == 0) go(phased_probe<1024, 8, 8, 0>, lds);
            else if (T == 256 && V == 16 && S == 16 && L == 0) go(phased_probe<256, 16, 16, 0>, lds);
            else { std::printf("{\"case\": \"%s\", \"error\": \"shape not built\"}\n", c.c_str()); continue; }
            moved = 2.0 * R * (double)chunks * T * V * 16;
        } else if (c.rfind("sweeps:", 0) == 0 && f.size() == 2) {
            const int K = f[0];
            const bool all = f[1] != 0;
            constexpr int T = 512, V = 16;
            const int64_t chunks = bytes / ((int64_t)T * V * 16);
            const int lds = 84 * 1024;                      // keeps a second workgroup off the CU
            auto go = [&](auto k) {
                CHECK(hipFuncSetAttribute(reinterpret_cast<const void*>(k), hipFuncAttributeMaxDynamicSharedMemorySize, lds));
                auto launch = [&]() {
                    CHECK(hipMemsetAsync(meet, 0, sizeof(Meet), 0));
                    hipLaunchKernelGGL(k, dim3(cus), dim3(T), (size_t)lds, 0, p, R, chunks, meet);
                    CHECK(hipGetLastError());
                };
                fill(); launch(); CHECK(hipDeviceSynchronize());
                // the sum wherever it was written, a rank's own value elsewhere
                const uint32_t sum = (uint32_t)R * (R + 1) / 2;
                const size_t cw = (size_t)T * V * 4;
                for (int r = 0; r < R && ok; r += std::max(1, R - 1)) {
                    CHECK(hipMemcpy(host.data(), p.p[r], bytes, hipMemcpyDeviceToHost));
                    for (int64_t ch = 0; ch < chunks && ok; ++ch)
                        for (size_t i = 0; i < cw; i += 251)
                            if (host[ch * cw + i] != ((all || ch % R == r) ? sum : (uint32_t)(r + 1))) { ok = false; break; }
                }
                fill();     // an allreduce in place would otherwise sum sums
                timed(launch);
                Meet hm; CHECK(hipMemcpy(&hm, meet, sizeof(hm), hipMemcpyDeviceToHost));
                if (hm.failed) ok = false;
            };
            if (K == 0 && all) go(sweeps_probe<1, true, false>);
            else if (K == 0) go(sweeps_probe<1, false, false>);
            else if (K == 1 && all) go(sweeps_probe<1, true, true>);
            else if (K == 1) go(sweeps_probe<1, false, true>);
            else if (K == 2 && all) go(sweeps_probe<2, true, true>);
            else if (K == 2) go(sweeps_probe<2, false, true>);
            else if (K == 3 && all) go(sweeps_probe<3, true, true>);
            else if (K == 3) go(sweeps_probe<3, false, true>);
            else { std::printf("{\"case\": \"%s\", \"error\": \"K must be 0 .. 3\"}\n", c.c_str()); continue; }
            moved = (double)(all ? 2 * R : R + 1) * (double)chunks * T * V * 16;
        } else if ((c.rfind("read:", 0) == 0 || c.rfind("write:", 0) == 0 || c.rfind("copy:", 0) == 0) && f.size() == 1) {
            const int T = f[0], kind = c[0] == 'r' ? 0 : c[0] == 'w' ? 1 : 2;
            if (T % 64 || T < 64 || T > 1024 || (kind == 2 && R % 2)) { std::printf("{\"case\": \"%s\", \"error\": \"shape not available\"}\n", c.c_str()); continue; }
            const int64_t tiles = bytes / ((int64_t)T * 16);
            int run = 256; while (run > 1 && 8 * run > tiles) run >>= 1;
            const int64_t grid = (tiles + 8 * run - 1) / (8 * run) * (8 * run);
            fill();
            timed([&]() { hipLaunchKernelGGL(stream_kernel, dim3((unsigned)grid), dim3(T), 0, 0, p, R, tiles, __builtin_ctz(run), kind, sink); CHECK(hipGetLastError()); });
            moved = (double)R * (double)tiles * T * 16;
        } else { std::printf("{\"case\": \"%s\", \"error\": \"unknown case\"}\n", c.c_str()); continue; }
        const float ms = total / reps;
        std::printf("{\"case\": \"%s\", \"ranks\": %d, \"bytes_per_rank\": %zu, \"verified\": %s, \"ms_avg\": %.4f, \"ms_min\": %.4f, \"hbm_bytes\": %.0f, \"GBps\": %.0f, \"frac_of_8TBps\": %.4f%s}\n",
                    c.c_str(), R, bytes, ok ? "true" : "false", ms, best, moved, moved / ms / 1e6, moved / ms / 1e6 / 8000.0, extra.c_str());
        std::fflush(stdout);
    }
    return 0;
}
