// gfx950 kernels of the executor: element arithmetic, the chunk reduce/copy primitives, the
// level runner, the persistent (flag-ordered) runner and the column runner.
//
// Arithmetic contract (what the reference's Vec<T>::operator+ computes on its hardware,
// csrc/plugins/cuda/kernel/vec.h:104-111,170-177,232-239): one correctly rounded addition in the
// storage type per element per reduce; NaN results are the canonical NaN (all mantissa bits set).
// bf16 is computed as RNE(float(a) + float(b)), which equals the single bf16 rounding because the
// float sum of two 8-bit-significand values is exact or rounds innocuously (24 >= 2*8+2).
#include <hip/hip_runtime.h>

#include <atomic>
#include <cstring>
#include <utility>

#include "kernels.h"

namespace pccl_hip {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef _Float16 h2 __attribute__((ext_vector_type(2)));

// Every pointer the kernels see is device memory: say so, so that global_* (not flat_*)
// instructions are selected.
#define PCCL_GLOBAL __attribute__((address_space(1)))
// Plan tables never change while a kernel runs: reading them through the constant address space
// lets uniform accesses become scalar loads (scalar cache, no vector-memory slot, no readfirstlane).
#define PCCL_CONST __attribute__((address_space(4)))
template <class T> __device__ __forceinline__ const PCCL_CONST T* as_const(const T* p) { return (const PCCL_CONST T*)p; }
template <class T> __device__ __forceinline__ T load_const(const T* p) {   // whole table record, 8 bytes at a time
    static_assert(sizeof(T) % 8 == 0, "table records are multiples of 8 bytes");
    T out;
    const PCCL_CONST uint64_t* w = (const PCCL_CONST uint64_t*)p;
    uint64_t* o = reinterpret_cast<uint64_t*>(&out);
#pragma unroll
    for (unsigned i = 0; i < sizeof(T) / 8; ++i) o[i] = w[i];
    return out;
}
constexpr int kThreads = 256;
constexpr int kMaxR = PCCL_HIP_MAX_VRANKS;

// ------------------------------------------------------------------------------- arithmetic

template <int DT> struct ElemBytes { static constexpr int value = (DT == PCCL_F32 || DT == PCCL_I32) ? 4 : (DT == PCCL_F16 || DT == PCCL_BF16) ? 2 : 1; };

__device__ __forceinline__ float as_f32(uint32_t u) { return __builtin_bit_cast(float, u); }
__device__ __forceinline__ uint32_t as_u32(float f) { return __builtin_bit_cast(uint32_t, f); }

// MAX / MIN are IEEE 754-2019 maximum / minimum: a NaN operand gives NaN (written canonically, like
// every NaN result here) and -0 orders below +0.  gfx950 has both as one instruction
// (v_maximum3_f32 / v_minimum3_f32 and their packed f16 forms).
template <int OP>
__device__ __forceinline__ float f32_comb(float a, float b) {
    if constexpr (OP == PCCL_SUM) return a + b;
    else if constexpr (OP == PCCL_MAX) return __builtin_elementwise_maximum(a, b);
    else return __builtin_elementwise_minimum(a, b);
}
template <int OP>
__device__ __forceinline__ h2 f16x2_comb(h2 a, h2 b) {
    if constexpr (OP == PCCL_SUM) return a + b;
    else if constexpr (OP == PCCL_MAX) return __builtin_elementwise_maximum(a, b);
    else return __builtin_elementwise_minimum(a, b);
}
__device__ __forceinline__ float f32_comb(float a, float b, int redop) {
    return redop == PCCL_SUM ? f32_comb<PCCL_SUM>(a, b) : redop == PCCL_MAX ? f32_comb<PCCL_MAX>(a, b) : f32_comb<PCCL_MIN>(a, b);
}

__device__ __forceinline__ uint32_t f32_op(uint32_t ua, uint32_t ub, int redop) {
    const float r = f32_comb(as_f32(ua), as_f32(ub), redop);
    return (r != r) ? 0x7FFFFFFFu : as_u32(r);
}

// float -> bf16 bits in the HIGH half of the result, round to nearest even, canonical NaN
__device__ __forceinline__ uint32_t bf16_round_hi(float f) {
    uint32_t u = as_u32(f);
    uint32_t r = u + 0x7FFFu + ((u >> 16) & 1u);
    return (f != f) ? 0x7FFF0000u : (r & 0xFFFF0000u);
}

__device__ __forceinline__ uint32_t bf16x2_op(uint32_t a, uint32_t b, int redop) {
    // a selected value is a bf16 already, so the rounding below only acts on sums
    float lo = f32_comb(as_f32(a << 16), as_f32(b << 16), redop);
    float hi = f32_comb(as_f32(a & 0xFFFF0000u), as_f32(b & 0xFFFF0000u), redop);
    return bf16_round_hi(hi) | (bf16_round_hi(lo) >> 16);
}

__device__ __forceinline__ uint32_t f16x2_op(uint32_t ua, uint32_t ub, int redop) {
    const h2 a = __builtin_bit_cast(h2, ua), b = __builtin_bit_cast(h2, ub);
    const h2 r = redop == PCCL_SUM ? f16x2_comb<PCCL_SUM>(a, b) : redop == PCCL_MAX ? f16x2_comb<PCCL_MAX>(a, b) : f16x2_comb<PCCL_MIN>(a, b);
    uint32_t u = __builtin_bit_cast(uint32_t, r);
    if (r[0] != r[0]) u = (u & 0xFFFF0000u) | 0x7FFFu;
    if (r[1] != r[1]) u = (u & 0x0000FFFFu) | 0x7FFF0000u;
    return u;
}

// fp8 (reference vec.h:272-426): widen both operands (exact), add with one f16 rounding, narrow
// with round-to-nearest-even and saturation to the largest finite value; NaN results are 0x7F.
// The conversion instructions of gfx950 implement the OCP formats (fp8 = E4M3, bf8 = E5M2); the
// saturation is done here with a clamp so that it does not depend on the overflow mode bit.
typedef float f32x2 __attribute__((ext_vector_type(2)));

template <bool E5M2, bool HI>
__device__ __forceinline__ uint32_t fp8_pair_op(uint32_t x, uint32_t y, uint32_t out, int redop) {
    constexpr float kMax = E5M2 ? 57344.0f : 448.0f;
    f32x2 a, b;
    if constexpr (E5M2) { a = __builtin_amdgcn_cvt_pk_f32_bf8(x, HI); b = __builtin_amdgcn_cvt_pk_f32_bf8(y, HI); }
    else { a = __builtin_amdgcn_cvt_pk_f32_fp8(x, HI); b = __builtin_amdgcn_cvt_pk_f32_fp8(y, HI); }
    float r0, r1;
    if (redop == PCCL_SUM) {
        // the float sum of two f16-representable values rounds to f16 exactly as their f16 sum
        r0 = (float)(_Float16)(a.x + b.x);
        r1 = (float)(_Float16)(a.y + b.y);
    } else {
        r0 = f32_comb(a.x, b.x, redop); r1 = f32_comb(a.y, b.y, redop);
    }
    const bool n0 = r0 != r0, n1 = r1 != r1;
    r0 = n0 ? 0.0f : __builtin_fminf(__builtin_fmaxf(r0, -kMax), kMax);
    r1 = n1 ? 0.0f : __builtin_fminf(__builtin_fmaxf(r1, -kMax), kMax);
    if constexpr (E5M2) out = __builtin_amdgcn_cvt_pk_bf8_f32(r0, r1, out, HI);
    else out = __builtin_amdgcn_cvt_pk_fp8_f32(r0, r1, out, HI);
    constexpr int sh = HI ? 16 : 0;
    if (n0) out = (out & ~(0xFFu << sh)) | (0x7Fu << sh);
    if (n1) out = (out & ~(0xFF00u << sh)) | (0x7F00u << sh);
    return out;
}

template <bool E5M2>
__device__ __forceinline__ uint32_t fp8x4_op(uint32_t a, uint32_t b, int redop) {
    uint32_t out = 0;
    out = fp8_pair_op<E5M2, false>(a, b, out, redop);
    out = fp8_pair_op<E5M2, true>(a, b, out, redop);
    return out;
}

__device__ __forceinline__ uint32_t i32_op(uint32_t a, uint32_t b, int redop) {
    if (redop == PCCL_SUM) return a + b;
    int x = (int)a, y = (int)b;
    return (uint32_t)(redop == PCCL_MAX ? (x > y ? x : y) : (x < y ? x : y));
}

template <int DT>
__device__ __forceinline__ uint32_t word_op(uint32_t a, uint32_t b, int redop) {
    if constexpr (DT == PCCL_F32) return f32_op(a, b, redop);
    else if constexpr (DT == PCCL_I32) return i32_op(a, b, redop);
    else if constexpr (DT == PCCL_BF16) return bf16x2_op(a, b, redop);
    else if constexpr (DT == PCCL_F16) return f16x2_op(a, b, redop);
    else if constexpr (DT == PCCL_F8E4M3) return fp8x4_op<false>(a, b, redop);
    else return fp8x4_op<true>(a, b, redop);
}

template <int DT>
__device__ __forceinline__ u32x4 vec_op_words(u32x4 a, u32x4 b, int redop) {
    u32x4 r;
    r.x = word_op<DT>(a.x, b.x, redop);
    r.y = word_op<DT>(a.y, b.y, redop);
    r.z = word_op<DT>(a.z, b.z, redop);
    r.w = word_op<DT>(a.w, b.w, redop);
    return r;
}

// Whole vectors take a shorter road than word_op: the arithmetic runs as if no NaN could
// come out, one unordered compare per pair of results notes whether one did, and only lanes that
// saw one go back and canonicalise (rare: the branch is skipped by the whole wave otherwise).
// The results are those of word_op bit for bit.  bf16 rounds with v_cvt_pk_bf16_f32, which was
// checked on this GPU against the integer form of bf16_round_hi for every non-NaN float.
typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));

template <int DT, int OP>
__device__ __forceinline__ u32x4 vec_fast(u32x4 a, u32x4 b) {
    if constexpr (DT == PCCL_F32) {
        const float r0 = f32_comb<OP>(as_f32(a.x), as_f32(b.x)), r1 = f32_comb<OP>(as_f32(a.y), as_f32(b.y));
        const float r2 = f32_comb<OP>(as_f32(a.z), as_f32(b.z)), r3 = f32_comb<OP>(as_f32(a.w), as_f32(b.w));
        u32x4 r = {as_u32(r0), as_u32(r1), as_u32(r2), as_u32(r3)};
        // one compare per pair of results, combined on the scalar side: the whole wave takes the
        // repair branch if any lane saw a NaN (the repairs themselves are per element)
        if (__builtin_expect((__builtin_amdgcn_ballot_w64(__builtin_isunordered(r0, r1)) | __builtin_amdgcn_ballot_w64(__builtin_isunordered(r2, r3))) != 0, 0)) {
            if (r0 != r0) r.x = 0x7FFFFFFFu;
            if (r1 != r1) r.y = 0x7FFFFFFFu;
            if (r2 != r2) r.z = 0x7FFFFFFFu;
            if (r3 != r3) r.w = 0x7FFFFFFFu;
        }
        return r;
    } else if constexpr (DT == PCCL_BF16) {
        // word by word, no arrays: everything stays in registers whatever the surrounding code looks like
        uint64_t nan = 0;
        auto word = [&](uint32_t x, uint32_t y) {
            const float lo = f32_comb<OP>(as_f32(x << 16), as_f32(y << 16));
            const float hi = f32_comb<OP>(as_f32(x & 0xFFFF0000u), as_f32(y & 0xFFFF0000u));
            nan |= __builtin_amdgcn_ballot_w64(__builtin_isunordered(lo, hi));
            const f32x2 pair = {lo, hi};
            return __builtin_bit_cast(uint32_t, __builtin_convertvector(pair, bf16x2_t));
        };
        auto repair = [](uint32_t w) {
            if ((w & 0x7FFFu) > 0x7F80u) w = (w & 0xFFFF0000u) | 0x7FFFu;
            if ((w & 0x7FFF0000u) > 0x7F800000u) w = (w & 0x0000FFFFu) | 0x7FFF0000u;
            return w;
        };
        u32x4 r = {word(a.x, b.x), word(a.y, b.y), word(a.z, b.z), word(a.w, b.w)};
        if (__builtin_expect(nan != 0, 0)) { r.x = repair(r.x); r.y = repair(r.y); r.z = repair(r.z); r.w = repair(r.w); }
        return r;
    } else if constexpr (DT == PCCL_F16) {
        uint64_t nan = 0;
        auto word = [&](uint32_t x, uint32_t y) {
            const h2 s = f16x2_comb<OP>(__builtin_bit_cast(h2, x), __builtin_bit_cast(h2, y));
            nan |= __builtin_amdgcn_ballot_w64(__builtin_isunordered(s[0], s[1]));
            return __builtin_bit_cast(uint32_t, s);
        };
        auto repair = [](uint32_t w) {
            if ((w & 0x7FFFu) > 0x7C00u) w = (w & 0xFFFF0000u) | 0x7FFFu;
            if ((w & 0x7FFF0000u) > 0x7C000000u) w = (w & 0x0000FFFFu) | 0x7FFF0000u;
            return w;
        };
        u32x4 r = {word(a.x, b.x), word(a.y, b.y), word(a.z, b.z), word(a.w, b.w)};
        if (__builtin_expect(nan != 0, 0)) { r.x = repair(r.x); r.y = repair(r.y); r.z = repair(r.z); r.w = repair(r.w); }
        return r;
    } else {
        return vec_op_words<DT>(a, b, OP);
    }
}

// The arithmetic of vec_fast with nothing done about NaN results, and the canonicalisation as a step
// of its own.  A NaN never turns back into a number under SUM, MAX or MIN (IEEE 754-2019 maximum and
// minimum propagate it, as addition does, and the bf16 rounding keeps a quiet NaN a NaN), so a chain or
// tree of these operations gives a NaN at its end exactly when one of its steps did, and making only the
// end result canonical gives the bits that canonicalising after every step gives.  The read phases of
// the phased runner use this: their loops then hold no branch, and the loads of the next vectors are
// not held up behind a test of this one's result.  Not for a value that no operation produced (a
// copied NaN keeps its payload), and not for the 8-bit floats (their clamp would lose a NaN).
template <int DT, int OP>
__device__ __forceinline__ u32x4 vec_bare(u32x4 a, u32x4 b) {
    if constexpr (DT == PCCL_F32) {
        return u32x4{as_u32(f32_comb<OP>(as_f32(a.x), as_f32(b.x))), as_u32(f32_comb<OP>(as_f32(a.y), as_f32(b.y))),
                     as_u32(f32_comb<OP>(as_f32(a.z), as_f32(b.z))), as_u32(f32_comb<OP>(as_f32(a.w), as_f32(b.w)))};
    } else if constexpr (DT == PCCL_BF16) {
        auto word = [](uint32_t x, uint32_t y) {
            const f32x2 pair = {f32_comb<OP>(as_f32(x << 16), as_f32(y << 16)), f32_comb<OP>(as_f32(x & 0xFFFF0000u), as_f32(y & 0xFFFF0000u))};
            return __builtin_bit_cast(uint32_t, __builtin_convertvector(pair, bf16x2_t));
        };
        return u32x4{word(a.x, b.x), word(a.y, b.y), word(a.z, b.z), word(a.w, b.w)};
    } else if constexpr (DT == PCCL_F16) {
        auto word = [](uint32_t x, uint32_t y) {
            return __builtin_bit_cast(uint32_t, f16x2_comb<OP>(__builtin_bit_cast(h2, x), __builtin_bit_cast(h2, y)));
        };
        return u32x4{word(a.x, b.x), word(a.y, b.y), word(a.z, b.z), word(a.w, b.w)};
    } else {
        return vec_fast<DT, OP>(a, b);
    }
}
// f32 and f16 chains and trees run with the deferred form (16-rank halving-doubling 0.762 -> 0.786 of
// peak, 32-rank f32 MAX 0.796 -> 0.840, f16 reduce_scatter 0.800 -> 0.807).  bf16 keeps the test per
// step: its arithmetic is seven instructions per element pair, and without a branch after every vector
// the compiler gathers the arithmetic of a whole rank behind that rank's last fetch, where no fetch
// overlaps it (headline 0.791 -> 0.767; with the arithmetic pinned after each group of fetches 0.781).
template <int DT> constexpr bool kDeferredNan = DT == PCCL_F32 || DT == PCCL_F16;
template <int DT, int OP>
__device__ __forceinline__ u32x4 vec_phase(u32x4 a, u32x4 b) {
    if constexpr (kDeferredNan<DT>) return vec_bare<DT, OP>(a, b); else return vec_fast<DT, OP>(a, b);
}

template <int DT>
__device__ __forceinline__ u32x4 canon_nan(u32x4 r) {
    if constexpr (DT == PCCL_F32) {
        auto word = [](uint32_t w) { return (w & 0x7FFFFFFFu) > 0x7F800000u ? 0x7FFFFFFFu : w; };
        return u32x4{word(r.x), word(r.y), word(r.z), word(r.w)};
    } else if constexpr (DT == PCCL_BF16 || DT == PCCL_F16) {
        constexpr uint32_t inf = DT == PCCL_BF16 ? 0x7F80u : 0x7C00u;
        auto word = [](uint32_t w) {
            if ((w & 0x7FFFu) > inf) w = (w & 0xFFFF0000u) | 0x7FFFu;
            if ((w & 0x7FFF0000u) > (inf << 16)) w = (w & 0x0000FFFFu) | 0x7FFF0000u;
            return w;
        };
        return u32x4{word(r.x), word(r.y), word(r.z), word(r.w)};
    } else {
        return r;
    }
}

// One decision on the operator per vector: each branch below inlines the word code with a
// constant operator, so the four words run back to back without tests in between.
template <int DT>
__device__ __forceinline__ u32x4 vec_op(u32x4 a, u32x4 b, int redop) {
    if (redop == PCCL_SUM) return vec_fast<DT, PCCL_SUM>(a, b);
    if (redop == PCCL_MAX) return vec_fast<DT, PCCL_MAX>(a, b);
    return vec_fast<DT, PCCL_MIN>(a, b);
}

// one element at byte address granularity (heads, tails, partial vectors, misaligned ranges)
template <int DT>
__device__ __forceinline__ uint32_t load_elem(const char* p) {
    constexpr int ES = ElemBytes<DT>::value;
    if constexpr (ES == 4) return *(const PCCL_GLOBAL uint32_t*)(p);
    else if constexpr (ES == 2) return *(const PCCL_GLOBAL uint16_t*)(p);
    else return *(const PCCL_GLOBAL uint8_t*)(p);
}
template <int DT>
__device__ __forceinline__ void store_elem(char* p, uint32_t v) {
    constexpr int ES = ElemBytes<DT>::value;
    if constexpr (ES == 4) *(PCCL_GLOBAL uint32_t*)(p) = v;
    else if constexpr (ES == 2) *(PCCL_GLOBAL uint16_t*)(p) = (uint16_t)v;
    else *(PCCL_GLOBAL uint8_t*)(p) = (uint8_t)v;
}
template <int DT>
__device__ __forceinline__ uint32_t elem_op(uint32_t a, uint32_t b, int redop) {
    // 2-byte types ride in the low half of a word; the zero high halves reduce to zero
    return word_op<DT>(a, b, redop);
}

typedef const PCCL_GLOBAL u32x4* gvec_cptr;
typedef PCCL_GLOBAL u32x4* gvec_ptr;
__device__ __forceinline__ u32x4 ldv(const char* p) { return *(gvec_cptr)(p); }
__device__ __forceinline__ void stv(char* p, u32x4 v) { *(gvec_ptr)(p) = v; }
// Streaming variants for data touched once.  Two forms, both measured on MI355X:
//  * pointer form: used by the column runners, whose per-store scalar work matters (building a
//    buffer descriptor per store cost the 32-rank tree 5 %, and the ring is the same either way).
//    Loads are non-temporal (nt; agent scope on top changes nothing for them).  Stores are nt sc1
//    like those of the buffer form below: programs that mostly write gain from the agent-scope bit
//    (8-rank allgather as one launch on the caller's tensors, 512 MB per rank 0.91 -> 0.81 ms,
//    16 MB per rank 31 -> 24 us), programs that read as much as they write are the same either way
//    (headline ring, halving-doubling, tree, reduce_scatter).  The compiler has no builtin for a
//    pointer store with that bit, hence the asm; the s_nop gives the one wait state that a 128-bit
//    store needs before a vector instruction may overwrite its data registers, which the compiler
//    inserts for stores it knows and cannot for this one;
//  * raw buffer operations (wave-uniform base in a resource descriptor, 32-bit byte offset per
//    lane) marked non-temporal AND agent scope (nt sc1): used by everything built on range_op.
//    Headline graph with the level runner: cached 3.22 ms, sc1 3.18, nt 3.06 (as global or as
//    buffer operations alike), nt sc1 2.99; plain copy 6.28 -> 6.55 TB/s.  The agent-scope bit also
//    makes the access coherent across the XCDs' L2s (a store is written through before it is
//    acknowledged, a load does not hit a stale line), which the persistent runner relies on.
__device__ __forceinline__ u32x4 ldv_nt(const char* p) { return __builtin_nontemporal_load((gvec_cptr)(p)); }
__device__ __forceinline__ void stv_nt(char* p, u32x4 v) {
    asm volatile("global_store_dwordx4 %0, %1, off sc1 nt\n\ts_nop 0" : : "v"((gvec_ptr)(p)), "v"(v) : "memory");
}
constexpr int kAuxStream = 16 | 2;   // sc1 | nt
__device__ __forceinline__ __amdgpu_buffer_rsrc_t stream_rsrc(const char* uniform_base) {
    return __builtin_amdgcn_make_buffer_rsrc((void*)uniform_base, 0, 0x7FFFFFFF, 0x00020000);
}

// ------------------------------------------------------------------------------- range primitives
//
// c[i] = a[i] (op) b[i] (IS_REDUCE) or c[i] = a[i], i in [0, n) elements, cooperatively by
// `nthreads` threads.  Any alignment: when the three addresses are congruent modulo 16 the body runs
// as 128-bit loads and stores with a scalar head and tail; otherwise element by element.
//
// How memory is touched is a policy: cached (plain global accesses) or streaming (the nt sc1 buffer
// operations above, which are also what makes data handed from one workgroup to another through a
// flag visible without writing back or invalidating whole caches).

enum { MEM_CACHED = 0, MEM_STREAM = 1, MEM_COHERENT = 1 };

template <int POLICY>
struct Mem {     // MEM_CACHED
    const char* base;
    __device__ __forceinline__ explicit Mem(const char* b) : base(b) {}
    __device__ __forceinline__ u32x4 ldv(int64_t off) const { return ::pccl_hip::ldv(base + off); }
    __device__ __forceinline__ void stv(int64_t off, u32x4 v) const { ::pccl_hip::stv((char*)base + off, v); }
    template <int DT> __device__ __forceinline__ uint32_t lde(int64_t off) const { return load_elem<DT>(base + off); }
    template <int DT> __device__ __forceinline__ void ste(int64_t off, uint32_t x) const { store_elem<DT>((char*)base + off, x); }
};

template <>
struct Mem<MEM_STREAM> {
    __amdgpu_buffer_rsrc_t rs;
    __device__ __forceinline__ explicit Mem(const char* b) : rs(stream_rsrc(b)) {}
    __device__ __forceinline__ u32x4 ldv(int64_t off) const { return __builtin_amdgcn_raw_buffer_load_b128(rs, (int)off, 0, kAuxStream); }
    __device__ __forceinline__ void stv(int64_t off, u32x4 v) const { __builtin_amdgcn_raw_buffer_store_b128(v, rs, (int)off, 0, kAuxStream); }
    template <int DT> __device__ __forceinline__ uint32_t lde(int64_t off) const {
        constexpr int ES = ElemBytes<DT>::value;
        if constexpr (ES == 4) return __builtin_amdgcn_raw_buffer_load_b32(rs, (int)off, 0, kAuxStream);
        else if constexpr (ES == 2) return __builtin_amdgcn_raw_buffer_load_b16(rs, (int)off, 0, kAuxStream);
        else return __builtin_amdgcn_raw_buffer_load_b8(rs, (int)off, 0, kAuxStream);
    }
    template <int DT> __device__ __forceinline__ void ste(int64_t off, uint32_t x) const {
        constexpr int ES = ElemBytes<DT>::value;
        if constexpr (ES == 4) __builtin_amdgcn_raw_buffer_store_b32(x, rs, (int)off, 0, kAuxStream);
        else if constexpr (ES == 2) __builtin_amdgcn_raw_buffer_store_b16((uint16_t)x, rs, (int)off, 0, kAuxStream);
        else __builtin_amdgcn_raw_buffer_store_b8((uint8_t)x, rs, (int)off, 0, kAuxStream);
    }
};

// The ranges handed to the streaming form must be shorter than 2 GiB (offsets are 32-bit) and their
// base addresses wave-uniform.
template <int DT, bool IS_REDUCE, int POLICY = MEM_STREAM>
__device__ __forceinline__ void range_op(const char* a, const char* b, char* c, int64_t n, int redop,
                                         int tid, int nthreads) {
    constexpr int ES = ElemBytes<DT>::value;
    constexpr int VE = 16 / ES;
    const Mem<POLICY> A(a), B(b), C(c);
    uintptr_t ua = (uintptr_t)a, ub = (uintptr_t)b, uc = (uintptr_t)c;
    bool congruent = ((ua ^ uc) & 15) == 0 && (!IS_REDUCE || ((ub ^ uc) & 15) == 0);
    if (!congruent) {
        for (int64_t i = tid; i < n; i += nthreads) {
            uint32_t x = A.template lde<DT>(i * ES);
            if constexpr (IS_REDUCE) x = elem_op<DT>(x, B.template lde<DT>(i * ES), redop);
            C.template ste<DT>(i * ES, x);
        }
        return;
    }
    int64_t head = (int64_t)(((16 - (uc & 15)) & 15) / ES);
    if (head > n) head = n;
    if (tid < head) {
        uint32_t x = A.template lde<DT>((int64_t)tid * ES);
        if constexpr (IS_REDUCE) x = elem_op<DT>(x, B.template lde<DT>((int64_t)tid * ES), redop);
        C.template ste<DT>((int64_t)tid * ES, x);
    }
    const int64_t h = head * ES;   // byte offset of the vector body
    n -= head;
    int64_t nvec = n / VE;
    int64_t v = tid;
    // 4 vectors per thread per trip: all loads issued before the first store
    for (; v + 3 * (int64_t)nthreads < nvec; v += 4 * (int64_t)nthreads) {
        const int64_t o0 = h + v * 16, o1 = h + (v + nthreads) * 16, o2 = h + (v + 2 * nthreads) * 16, o3 = h + (v + 3 * nthreads) * 16;
        u32x4 x0 = A.ldv(o0), x1 = A.ldv(o1), x2 = A.ldv(o2), x3 = A.ldv(o3);
        if constexpr (IS_REDUCE) {
            u32x4 y0 = B.ldv(o0), y1 = B.ldv(o1), y2 = B.ldv(o2), y3 = B.ldv(o3);
            x0 = vec_op<DT>(x0, y0, redop); x1 = vec_op<DT>(x1, y1, redop); x2 = vec_op<DT>(x2, y2, redop); x3 = vec_op<DT>(x3, y3, redop);
        }
        C.stv(o0, x0); C.stv(o1, x1); C.stv(o2, x2); C.stv(o3, x3);
    }
    for (; v < nvec; v += nthreads) {
        u32x4 x = A.ldv(h + v * 16);
        if constexpr (IS_REDUCE) x = vec_op<DT>(x, B.ldv(h + v * 16), redop);
        C.stv(h + v * 16, x);
    }
    int64_t tail0 = nvec * VE;
    for (int64_t i = tail0 + tid; i < n; i += nthreads) {
        uint32_t x = A.template lde<DT>(h + i * ES);
        if constexpr (IS_REDUCE) x = elem_op<DT>(x, B.template lde<DT>(h + i * ES), redop);
        C.template ste<DT>(h + i * ES, x);
    }
}

// byte copy with the same structure (used by copies of every dtype and by staging)
template <int POLICY = MEM_STREAM>
__device__ __forceinline__ void range_copy_bytes(const char* a, char* c, int64_t nbytes, int tid, int nthreads) {
    range_op<PCCL_F8E4M3, false, POLICY>(a, nullptr, c, nbytes, 0, tid, nthreads);
}

template <int DT>
__device__ __forceinline__ void range_dispatch(bool is_reduce, const char* a, const char* b, char* c, int64_t n,
                                               int redop, int tid, int nthreads) {
    if (is_reduce) range_op<DT, true>(a, b, c, n, redop, tid, nthreads);
    else range_copy_bytes(a, c, n * ElemBytes<DT>::value, tid, nthreads);
}

// ------------------------------------------------------------------------------- standalone primitives

// One workgroup per 4 KiB tile (one 128-bit vector per thread) and no grid-stride loop: measured
// on MI355X a plain copy runs at 6.6 TB/s this way against 5.0 TB/s with 64 KiB tiles walked by a
// capped persistent grid.
constexpr int64_t kPrimTileBytes = 4 * 1024;

// Which tile a workgroup takes.  Workgroups are dispatched round-robin over the 8 XCDs (workgroup
// w runs on XCD w % 8), and each XCD has its own L2.  Tiles are dealt to the XCDs in runs of
// `run` consecutive tiles: launch indices [k * 8 * run, (k + 1) * 8 * run) cover the same range
// of tiles, XCD x taking tiles [x * run, (x + 1) * run) of it.  All eight XCDs thus sweep one
// narrow window of memory together while each streams through whole neighbourhoods.  Measured on
// the headline graph: column program (4 KiB per rank and tile) run 1 (tiles interleaved) 1.637 ms,
// 8 1.629, 64 1.471, 128 1.409, 256 1.396, 512 1.394, 1024 1.420, one run per XCD 1.421; level
// runner (4 KiB pieces) run 1 3.087 ms, 8 2.918, 16 to 256 2.86 to 2.88, 1024 2.94, 4096 2.96;
// 4 GiB reduce 6.42 TB/s at run 1, 6.61 at 256; a plain copy does not care (6.6 to 6.8 TB/s).
// Other shapes (rings of 16 and 32 ranks, halving-doubling, trees) are as fast or faster at 256
// than at 1 or 16 with two exceptions of 4 to 7 %: a 16-rank bf16 ring of 128 MiB per rank and
// the 32-rank tree on ragged pieces, which like runs of 1 to 4 best.
// The mapping is a bijection on [0, round_up(tiles, 8 * run)); the caller skips what falls beyond.
constexpr int kXcds = 8;
constexpr int kXcdRun = 256;
// `run` is a power of two, so all of this is shifts and masks (a 64-bit division by a run-time
// value would be some forty scalar instructions in front of every workgroup's first load).
__host__ __device__ __forceinline__ int64_t span_tiles(int64_t tiles, int run) {
    const int64_t span = (int64_t)kXcds * run;
    return (tiles + span - 1) & ~(span - 1);
}
__device__ __forceinline__ int64_t xcd_tile(int64_t w, int run) {
    const int shift = __builtin_ctz((unsigned)run);
    const int64_t in = w & ((int64_t)kXcds * run - 1);
    return w - in + ((in & (kXcds - 1)) << shift) + (in >> 3);
}
static_assert(kXcds == 8 && (kXcdRun & (kXcdRun - 1)) == 0, "xcd_tile shifts by 3 and by log2(run)");

// Tiles are anchored at multiples of 4 KiB of the destination address, not at the start of the
// range: a range that starts at an odd address has ragged tiles at its two ends only.
template <int DT>
__global__ __launch_bounds__(kThreads) void reduce_kernel(const char* a, const char* b, char* c, int64_t n, int redop, int run) {
    constexpr int ES = ElemBytes<DT>::value;
    constexpr int64_t TE = kPrimTileBytes / ES;
    const int64_t lead = (int64_t)((uintptr_t)c % kPrimTileBytes) / ES;
    const int64_t ntiles = (n + lead + TE - 1) / TE;
    for (int64_t w = blockIdx.x; w < span_tiles(ntiles, run); w += gridDim.x) {
        const int64_t t = xcd_tile(w, run);
        if (t >= ntiles) continue;
        int64_t e0 = t * TE - lead, e1 = e0 + TE;
        if (e0 < 0) e0 = 0;
        if (e1 > n) e1 = n;
        range_op<DT, true>(a + e0 * ES, b + e0 * ES, c + e0 * ES, e1 - e0, redop, threadIdx.x, kThreads);
    }
}

__device__ __forceinline__ void copy_tiles(const char* src, char* dst, int64_t nbytes, int run) {
    const int64_t lead = (int64_t)((uintptr_t)dst % kPrimTileBytes);
    const int64_t ntiles = (nbytes + lead + kPrimTileBytes - 1) / kPrimTileBytes;
    for (int64_t w = blockIdx.x; w < span_tiles(ntiles, run); w += gridDim.x) {
        const int64_t t = xcd_tile(w, run);
        if (t >= ntiles) continue;
        int64_t b0 = t * kPrimTileBytes - lead, b1 = b0 + kPrimTileBytes;
        if (b0 < 0) b0 = 0;
        if (b1 > nbytes) b1 = nbytes;
        range_copy_bytes(src + b0, dst + b0, b1 - b0, threadIdx.x, kThreads);
    }
}

__global__ __launch_bounds__(kThreads) void copy_kernel(const char* src, char* dst, int64_t nbytes, int run) {
    copy_tiles(src, dst, nbytes, run);
}

__global__ __launch_bounds__(kThreads) void stage_kernel(RankPtrs src, RankPtrs dst, StageOffsets off, int64_t nbytes, int run) {
    const int r = blockIdx.y;
    copy_tiles(src.p[r] + off.src[r], dst.p[r] + off.dst[r], nbytes, run);
}

// A list of independent copies between rank tensors in one launch (the staged alltoall call composed
// into direct copies): workgroup w finds its copy by binary search over the tile prefix sums.
// (When all copies have the same number of tiles - an alltoall's chunks - the search is one
// division: a workgroup here moves 4 KiB, and the six dependent table reads of the search in front
// of that cost 8 x 256 MiB 13 % of its time, 0.76 against 0.66 ms.  The level runner's one extra
// table read, item -> op, is not worth replacing the same way: measured 0.5 % slower.)
__global__ __launch_bounds__(kThreads) void gather_kernel(const DevGatherCopy* copies, int n, int64_t total_tiles, int copy_tiles, RankPtrs src, RankPtrs dst, int run) {
    for (int64_t u = blockIdx.x; u < span_tiles(total_tiles, run); u += gridDim.x) {
        const int64_t w = xcd_tile(u, run);
        if (w >= total_tiles) continue;
        int lo = 0;
        if (copy_tiles > 0) {
            const uint32_t per = (uint32_t)copy_tiles;
            lo = (per & (per - 1)) == 0 ? (int)((uint32_t)w >> __builtin_ctz(per)) : (int)((uint32_t)w / per);
        } else {
            int hi = n;
            while (hi - lo > 1) {
                int mid = (lo + hi) >> 1;
                if (as_const(copies)[mid].first_tile <= w) lo = mid; else hi = mid;
            }
        }
        const DevGatherCopy c = load_const(copies + lo);
        const int64_t b0 = (w - c.first_tile) * kPrimTileBytes;
        const int64_t cnt = c.bytes - b0 < kPrimTileBytes ? c.bytes - b0 : kPrimTileBytes;
        range_copy_bytes(src.p[c.src_rank] + c.src_off + b0, dst.p[c.dst_rank] + c.dst_off + b0, cnt, threadIdx.x, kThreads);
    }
}

// Launch numbers.  Flags and ready words hold the number of the launch that last set them and are
// never cleared between launches, so every launch needs a number no earlier launch has left in them.
// The host counts 1, 2, ... up to kHostEpochLimit; launches recorded into a graph (whose arguments
// every replay repeats) take theirs from a device-side counter that starts at kGraphEpochBase, far
// from the host's range, and that this kernel advances in front of each of them.  Neither range
// runs out: the host clears the words and starts again from 1 when it reaches its limit, and this
// kernel does the same for its counter - all its threads clear the `nwords` flag and ready words
// behind the block, then the counter restarts at the base (`limit` is a parameter so that a test
// can bring the wrap within reach).
__global__ __launch_bounds__(kThreads) void advance_graph_epoch_kernel(StepState* state, int nwords, int32_t limit) {
    const int32_t e = state->graph_epoch;                 // every thread reads the same word
    int32_t next = (e < kGraphEpochBase ? kGraphEpochBase : e) + 1;
    if (next >= limit) {
        uint32_t* words = reinterpret_cast<uint32_t*>(state + 1);
        for (int i = threadIdx.x; i < nwords; i += kThreads) words[i] = 0;
        next = kGraphEpochBase + 1;
    }
    __syncthreads();                                      // all reads of the old value and all clears are done
    if (threadIdx.x == 0) __hip_atomic_store(&state->graph_epoch, next, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

__global__ __launch_bounds__(kThreads) void fill_zero_kernel(uint32_t* dst, int64_t nwords) {
    for (int64_t i = (int64_t)blockIdx.x * kThreads + threadIdx.x; i < nwords; i += (int64_t)gridDim.x * kThreads) dst[i] = 0;
}

// ------------------------------------------------------------------------------- level runner
//
// General path for any linked program: the data ops are grouped by dependency level and every
// level is one launch; the launch boundary orders the levels.  A workgroup runs whole (op, tile)
// items of its level.

template <int DT>
__global__ __launch_bounds__(kThreads) void level_kernel(StepwiseLaunch L, int item_begin, int item_end, int subs, int run, RankPtrs ptrs) {
    constexpr int ES = ElemBytes<DT>::value;
    constexpr int64_t SUB_ELEMS = kPrimTileBytes / ES;   // each workgroup takes one 4 KiB piece of an item
    const int tid = threadIdx.x;
    const int64_t total = (int64_t)(item_end - item_begin) * subs;
    for (int64_t u = blockIdx.x; u < span_tiles(total, run); u += gridDim.x) {
        const int64_t w = xcd_tile(u, run);
        if (w >= total) continue;
        int item;
        int64_t sub;
        if ((subs & (subs - 1)) == 0) {   // the usual case: item sizes are powers of two
            item = item_begin + (int)(w >> __builtin_ctz((unsigned)subs));
            sub = w & (subs - 1);
        } else {
            item = item_begin + (int)(w / subs);
            sub = w % subs;
        }
        int opi = as_const(L.item_op)[item];
        DevStepOp op = load_const(L.ops + opi);
        // items and pieces sit on a grid anchored `lead` elements in front of the op (see DevStepOp)
        int64_t e0 = (int64_t)(item - op.first_item) * L.tile_elems + sub * SUB_ELEMS - op.lead;
        int64_t e1 = e0 + SUB_ELEMS;
        const int64_t item_end = (int64_t)(item - op.first_item + 1) * L.tile_elems - op.lead;
        if (e1 > item_end) e1 = item_end;
        if (e1 > op.size) e1 = op.size;
        if (e0 < 0) e0 = 0;
        const int64_t cnt = e1 - e0;
        if (cnt <= 0) continue;
        char* self = ptrs.p[op.self()];
        const char* peer = ptrs.p[op.peer()];
        if (op.is_reduce())
            range_op<DT, true>(peer + (op.off0 + e0) * ES, self + (op.off1 + e0) * ES, self + (op.off2 + e0) * ES, cnt, op.redop(), tid, kThreads);
        else
            range_copy_bytes(peer + (op.off0 + e0) * ES, self + (op.off1 + e0) * ES, cnt * ES, tid, kThreads);
    }
}

// ------------------------------------------------------------------------------- persistent runner
//
// One persistent launch executes every data op of the linked program.  Work items are (op, tile)
// pairs in level order, dealt round-robin to the workgroups: workgroup b runs items b, b + G,
// b + 2G, ... in that order, waits before each until every item of the op's predecessors has been
// published, runs it, then publishes it.  An item only ever waits for items with smaller numbers,
// and every workgroup works through its items in increasing order, so the scheme cannot deadlock
// as long as all G workgroups are resident at once; the launcher sizes G from the occupancy the
// runtime reports.  (Handing out items through one atomic ticket counter instead cost about 90 ns
// per item - same-address atomics from 8 XCDs are serialised - which more than doubled the time
// of the headline graph.)
//
// Cross-workgroup visibility: one flag word per item and one "ready" word per op.  All data
// accesses of this kernel are agent-coherent (see Mem<MEM_COHERENT>), so handing an item over
// needs no cache-wide operation: every wave waits until its stores have been acknowledged, the
// workgroup meets at a barrier, and one thread publishes the item's flag with an agent-scope
// atomic store.  The workgroup that runs an op's first tile polls the flags of all tiles of all
// predecessors and then publishes the op's ready word; the op's other tiles (higher item numbers,
// so the ordering argument above still holds) wait for that one word.  (With every tile polling
// all the flags itself - a thousand words per predecessor at 16 KiB tiles - the polls were a sixth
// of the data traffic again, in coherent loads.  One completion counter per op, incremented by
// every finished tile, was worse still: same-address atomics serialise, 8.1 ms.  With cached data
// accesses and an agent-scope release / acquire fence per wave and item - a write-back and an
// invalidation of the XCD's whole L2 each - the headline graph took 16 ms.)  Flags and ready words
// hold the launch epoch, so they are never cleared.  Every wait is bounded by wall-clock time:
// when `timeout_ticks` of the 100 MHz counter have passed since the workgroup started, the waiter
// records (op, predecessor), and it and every workgroup that finds itself waiting afterwards leave
// before their next item, so the grid always drains and the host reports the stall as an error.
//
// Shape of the loop (it matters): the item number is a wave-uniform scalar, so the loop is
// controlled by scalar branches, and the single-thread blocks (stall check, publish) each sit
// between two barriers.  An earlier form claimed the item in a single-thread block at the top of
// the loop and published in another at the bottom, with no barrier between them across the back
// edge; the compiler merged the two blocks and let the other 255 threads run ahead into the next
// iteration's barrier while the claiming lane was masked off: they re-read the old item for ever
// and the launch never drained.

template <int DT>
__global__ __launch_bounds__(kThreads) __attribute__((amdgpu_waves_per_eu(8, 8)))
void persistent_kernel(StepwiseLaunch L, RankPtrs ptrs) {
    constexpr int ES = ElemBytes<DT>::value;
    __shared__ int s_stalled;   // set by a waiter that gave up (or saw that another workgroup had)
    int32_t* flags = reinterpret_cast<int32_t*>(L.state + 1);   // one per item
    int32_t* ready = flags + L.num_items;                       // one per op
    const int tid = threadIdx.x;
    const uint64_t t_start = __builtin_amdgcn_s_memrealtime();
    // The launch number that flags and ready words take: a kernel argument, or - for a launch
    // recorded into a graph, whose arguments every replay repeats - the device-side counter that
    // the one-thread kernel recorded in front of this one has just advanced.
    const int32_t epoch = L.epoch != 0 ? L.epoch
                                       : __hip_atomic_load(&L.state->graph_epoch, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    // A launch that works in a block shared between operations - a recorded launch may be replayed
    // long after it was recorded - first makes sure that the tables behind the block are still its
    // own: its item count, kernel arguments, would otherwise index another operation's tables.
    // Wave-uniform, before any barrier: every thread of every workgroup leaves.
    if (L.owner_tag != 0 && __hip_atomic_load(&L.state->owner, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != L.owner_tag) {
        if (blockIdx.x == 0 && tid == 0) __hip_atomic_store(&L.state->stale_owner, L.owner_tag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        return;
    }
    if (tid == 0) s_stalled = 0;
    __syncthreads();
    // The loop is software-pipelined over the workgroup's items: the descriptor of the next item and
    // (thread 0) a first look at its ready word are fetched while the current item's data is moving,
    // so that in the common case - the predecessors finished long ago - an item starts its loads
    // without a dependent chain of three memory round trips in front of them.
    int item = blockIdx.x;
    if (item >= L.num_items) return;
    int opi = as_const(L.item_op)[item];
    DevStepOp op = load_const(L.ops + opi);
    int32_t seen = 0;   // thread 0: the ready word of `op` as last read (0 = not read)
    for (;;) {
        const int next = item + (int)gridDim.x;
        const bool has_next = next < L.num_items;
        const int nopi = has_next ? as_const(L.item_op)[next] : 0;
        // wait (no barrier in here).  `word` is what this thread watches, `dep` who is late if it
        // never arrives.
        auto wait_for = [&](int32_t* word, int dep) {
            int nap = 1;
            while (__hip_atomic_load(word, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != epoch) {
                if (__builtin_amdgcn_s_memrealtime() - t_start > L.timeout_ticks) {
                    __hip_atomic_store(&L.state->error_dep, dep + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    __hip_atomic_store(&L.state->error_op, opi + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    s_stalled = 1;
                    return;
                }
                if (__hip_atomic_load(&L.state->error_op, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 0) { s_stalled = 1; return; }
                __builtin_amdgcn_s_sleep(1);
                for (int z = 1; z < nap; ++z) __builtin_amdgcn_s_sleep(8);
                if (nap < 4) nap <<= 1;   // at most about a microsecond between two looks
            }
        };
        const bool opens = item == op.first_item;   // wave-uniform
        if (opens) {
            // the op's first tile checks every tile of every predecessor: thread t watches items
            // t, t + 256, ... of each
            for (int k = 0; k < op.ndeps; ++k) {
                const int d = as_const(L.deps)[op.dep_start + k];
                const int first = as_const(L.ops)[d].first_item, nt = as_const(L.ops)[d].ntiles;
                for (int t = tid; t < nt; t += kThreads) wait_for(&flags[first + t], d);
            }
        } else if (tid == 0 && op.ndeps > 0 && seen != epoch) {
            // every other tile waits for the first tile's answer, one word
            wait_for(&ready[opi], as_const(L.deps)[op.dep_start]);
        }
        __syncthreads();   // everything this workgroup waited for has been seen; the data accesses
                           // below are agent-coherent, so no cache needs to be invalidated first
        const int stalled = __builtin_amdgcn_readfirstlane(s_stalled);
        if (stalled) break;   // a predecessor never arrived: do not touch the data, just leave
        if (opens && tid == 0 && op.ntiles > 1 && op.ndeps > 0)
            __hip_atomic_store(&ready[opi], epoch, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        DevStepOp nop = op;
        if (has_next) nop = load_const(L.ops + nopi);
        int64_t e0 = (int64_t)(item - op.first_item) * L.tile_elems - op.lead;
        int64_t e1 = e0 + L.tile_elems;
        if (e0 < 0) e0 = 0;
        if (e1 > op.size) e1 = op.size;
        const int64_t cnt = e1 - e0;
        char* self = ptrs.p[op.self()];
        const char* peer = ptrs.p[op.peer()];
        if (op.is_reduce())
            range_op<DT, true, MEM_COHERENT>(peer + (op.off0 + e0) * ES, self + (op.off1 + e0) * ES, self + (op.off2 + e0) * ES, cnt, op.redop(), tid, kThreads);
        else
            range_copy_bytes<MEM_COHERENT>(peer + (op.off0 + e0) * ES, self + (op.off1 + e0) * ES, cnt * ES, tid, kThreads);
        int32_t nseen = 0;
        if (tid == 0 && has_next && next != nop.first_item && nop.ndeps > 0)
            nseen = __hip_atomic_load(&ready[nopi], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        // every wave: its write-through stores have been acknowledged (they are visible to the
        // whole device) before the workgroup meets and one thread publishes the item
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();
        if (tid == 0) __hip_atomic_store(&flags[item], epoch, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __syncthreads();   // keeps the single-thread block away from the back edge (see above)
        if (!has_next) break;
        item = next; opi = nopi; op = nop; seen = nseen;
    }
}

// ------------------------------------------------------------------------------- column runner
//
// When every data op reads and writes the same element positions in all buffers, the program
// decomposes by position: what happens to position p involves only position p of the R buffers.
// A segment is a maximal position range with one op list; a workgroup takes a tile of a segment
// and runs the segment's column program on it start to finish, each thread on its own 16-byte
// vectors.  No workgroup ever depends on another, so there are no flags and no fences; values
// that the next instruction needs stay in registers (SRC_ACC) and writes that are overwritten
// before anything re-reads them are dropped (store == 0).  Results are bit-identical to running
// the ops one at a time in schedule order: every element sees the same operations in the same
// order with the same per-step rounding.

struct ColInstrDev { uint8_t self, peer, a_src, b_src, redop, store, a_first, b_first; };

__device__ __forceinline__ ColInstrDev unpack_instr(uint64_t w) {
    ColInstrDev i;
    i.self = w & 0xFF; i.peer = (w >> 8) & 0xFF; i.a_src = (w >> 16) & 0xFF; i.b_src = (w >> 24) & 0xFF;
    i.redop = (w >> 32) & 0xFF; i.store = (w >> 40) & 0xFF; i.a_first = (w >> 48) & 0xFF; i.b_first = (w >> 56) & 0xFF;
    return i;
}

// Store one value to the same position of every rank in `mask` (the broadcast tail of a program).
// Four rank pointers are fetched per round so that their scalar loads overlap.
template <bool NT>
__device__ __forceinline__ void broadcast_store(uint64_t mask, const RankPtrs& ptrs, int64_t off, u32x4 v) {
    while (mask) {
        int r[4];
        int n = 0;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            r[i] = mask ? __builtin_ctzll(mask) : 0;
            if (mask) { mask &= mask - 1; n = i + 1; }
        }
        char* p[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) p[i] = ptrs.p[r[i]];
#pragma unroll
        for (int i = 0; i < 4; ++i)
            if (i < n) { if (NT) stv_nt(p[i] + off, v); else stv(p[i] + off, v); }
    }
}

template <int DT, int U, bool NT>
__device__ __forceinline__ void column_tile(const PCCL_CONST uint64_t* prog, int prog_len, uint64_t bcast_mask, const RankPtrs& s_ptr_tab, int64_t vfirst, int tid) {
    char* const* s_ptr = s_ptr_tab.p;   // kernel arguments: uniform indices become scalar loads
    int64_t off[U];
#pragma unroll
    for (int u = 0; u < U; ++u) off[u] = (vfirst + (int64_t)u * kThreads + tid) * 16;
    u32x4 acc[U];
#pragma unroll
    for (int u = 0; u < U; ++u) acc[u] = u32x4{0, 0, 0, 0};
    for (int k = 0; k < prog_len; ++k) {
        const ColInstrDev in = unpack_instr(prog[k]);
        char* self = s_ptr[in.self];
        u32x4 a[U];
        if (in.a_src == 2 /*SRC_ACC*/) {
#pragma unroll
            for (int u = 0; u < U; ++u) a[u] = acc[u];
        } else {
            const char* peer = s_ptr[in.peer + (in.a_first ? kMaxR : 0)];
#pragma unroll
            for (int u = 0; u < U; ++u) a[u] = NT ? ldv_nt(peer + off[u]) : ldv(peer + off[u]);
        }
        if (in.b_src != 0 /*reduce*/) {
            u32x4 b[U];
            if (in.b_src == 2) {
#pragma unroll
                for (int u = 0; u < U; ++u) b[u] = acc[u];
            } else {
                const char* own = s_ptr[in.self + (in.b_first ? kMaxR : 0)];
#pragma unroll
                for (int u = 0; u < U; ++u) b[u] = NT ? ldv_nt(own + off[u]) : ldv(own + off[u]);
            }
#pragma unroll
            for (int u = 0; u < U; ++u) acc[u] = vec_op<DT>(a[u], b[u], in.redop);
        } else {
#pragma unroll
            for (int u = 0; u < U; ++u) acc[u] = a[u];
        }
        if (in.store & 3) {
#pragma unroll
            for (int u = 0; u < U; ++u) { if (NT) stv_nt(self + off[u], acc[u]); else stv(self + off[u], acc[u]); }
        }
    }
    if (bcast_mask) {
#pragma unroll
        for (int u = 0; u < U; ++u) broadcast_store<NT>(bcast_mask, s_ptr_tab, off[u], acc[u]);
    }
}

// A tile that the segment boundary cuts: whole vectors inside the segment run the program on
// 16-byte accesses, cut vectors element by element; every value goes through memory.
template <int DT>
__device__ __forceinline__ void column_edge_tile(const DevColSegment& seg, const PCCL_CONST uint64_t* prog, const RankPtrs& ptrs,
                                                 int64_t vfirst, int64_t tile_v, int tid, int nthreads) {
    constexpr int ES = ElemBytes<DT>::value;
    constexpr int VE = 16 / ES;
    char* const* s_ptr = ptrs.p;
    for (int64_t v = vfirst + tid; v < vfirst + tile_v; v += nthreads) {
        int64_t e0 = v * VE, e1 = e0 + VE;
        if (e0 < seg.start) e0 = seg.start;
        if (e1 > seg.end) e1 = seg.end;
        if (e0 >= e1) continue;
        if (e1 - e0 == VE) {
            int64_t o = v * 16;
            u32x4 acc = u32x4{0, 0, 0, 0};
            for (int k = 0; k < seg.prog_len; ++k) {
                const ColInstrDev in = unpack_instr(prog[k]);
                u32x4 a = in.a_src == 2 ? acc : ldv(s_ptr[in.peer + (in.a_first ? kMaxR : 0)] + o);
                if (in.b_src != 0) {
                    u32x4 b = in.b_src == 2 ? acc : ldv(s_ptr[in.self + (in.b_first ? kMaxR : 0)] + o);
                    acc = vec_op<DT>(a, b, in.redop);
                } else acc = a;
                if (in.store & 3) stv(s_ptr[in.self] + o, acc);
            }
            for (uint64_t m = seg.bcast_mask; m; m &= m - 1) stv(s_ptr[__builtin_ctzll(m)] + o, acc);
        } else {
            for (int64_t e = e0; e < e1; ++e) {
                int64_t o = e * ES;
                uint32_t acc = 0;
                for (int k = 0; k < seg.prog_len; ++k) {
                    const ColInstrDev in = unpack_instr(prog[k]);
                    uint32_t a = in.a_src == 2 ? acc : load_elem<DT>(s_ptr[in.peer + (in.a_first ? kMaxR : 0)] + o);
                    if (in.b_src != 0) {
                        uint32_t b = in.b_src == 2 ? acc : load_elem<DT>(s_ptr[in.self + (in.b_first ? kMaxR : 0)] + o);
                        acc = elem_op<DT>(a, b, in.redop);
                    } else acc = a;
                    if (in.store & 3) store_elem<DT>(s_ptr[in.self] + o, acc);
                }
                for (uint64_t m = seg.bcast_mask; m; m &= m - 1) store_elem<DT>(s_ptr[__builtin_ctzll(m)] + o, acc);
            }
        }
    }
}

// Which segment a tile belongs to (uniform).  When all segments have the same number of tiles - the
// chunks of a ring, the halves of a halving-doubling schedule - that is a shift or a division;
// otherwise a binary search over the segments' first tiles, log2 dependent table reads in front of
// the workgroup's first load.
__device__ __forceinline__ int find_segment(const ColumnLaunch& L, int64_t tile) {
    if (L.seg_tiles > 0) {
        const uint32_t per = (uint32_t)L.seg_tiles;
        return (per & (per - 1)) == 0 ? (int)((uint32_t)tile >> __builtin_ctz(per)) : (int)((uint32_t)tile / per);
    }
    int lo = 0, hi = L.num_segs;
    while (hi - lo > 1) {
        int mid = (lo + hi) >> 1;
        if (as_const(L.segs)[mid].first_tile <= tile) lo = mid; else hi = mid;
    }
    return lo;
}

template <int DT, int U>
__global__ __launch_bounds__(kThreads) void column_kernel(ColumnLaunch L, RankPtrs ptrs) {
    constexpr int ES = ElemBytes<DT>::value;
    constexpr int VE = 16 / ES;
    constexpr int64_t TILE_V = (int64_t)kThreads * U;
    const int tid = threadIdx.x;

    // tiles are dealt to the XCDs in runs (see xcd_tile)
    for (int64_t w = blockIdx.x; w < span_tiles(L.total_tiles, L.xcd_run); w += gridDim.x) {
        const int64_t tile = xcd_tile(w, L.xcd_run);
        if (tile >= L.total_tiles) continue;
        const int lo = find_segment(L, tile);
        const DevColSegment seg = load_const(L.segs + lo);
        const int64_t vfirst = seg.first_vec + (tile - seg.first_tile) * TILE_V;
        const PCCL_CONST uint64_t* prog = as_const(L.instrs) + seg.prog_start;
        const bool interior = vfirst * VE >= seg.start && (vfirst + TILE_V) * VE <= seg.end;
        if (interior) {
            // A segment whose every load is a first touch and whose every live store is final is
            // pure streaming: run it with non-temporal accesses throughout (a separate loop
            // instance, so the cache-policy hints cannot be merged away with the cached forms).
            if (seg.streaming) column_tile<DT, U, true>(prog, seg.prog_len, seg.bcast_mask, ptrs, vfirst, tid);
            else column_tile<DT, U, false>(prog, seg.prog_len, seg.bcast_mask, ptrs, vfirst, tid);
        } else {
            column_edge_tile<DT>(seg, prog, ptrs, vfirst, TILE_V, tid, kThreads);
        }
    }
}

// ------------------------------------------------------------------------------- column runner, values kept in LDS
//
// The same segment programs, with every value the program reads more than once kept on chip:
// each thread owns one 16-byte LDS slot per rank (slot r of thread t holds the current value of
// rank r at the thread's position).  A tile first fetches every rank the program reads by first
// touch - up to 8 independent streaming loads in flight per thread - into the slots, then runs
// the program on the slots (MEM operands read a slot, a write that is read back later goes to its
// slot) and sends only the last value of each rank to memory.  Each rank buffer is therefore read
// at most once and written at most once per position whatever the shape of the program (chains,
// halving-doubling butterflies, trees).  A thread only ever touches its own slots, so no barrier
// is needed.  Results are bit-identical to the op-by-op execution for the same reason as above.

// Slot (rank r, vector v) of thread t in a workgroup of T threads with V vectors per thread sits at
// index (r * V + v) * T + t: consecutive lanes 16 bytes apart (conflict-free 128-bit accesses), and a
// wave's 64 lanes form the contiguous 1 KiB block that one direct-to-LDS load fills.
template <int N>
__device__ __forceinline__ void slot_fetch(uint64_t word, const RankPtrs& ptrs, u32x4* slots, int V, int v, int T, int tid, int64_t off) {
    u32x4 x[N];
#pragma unroll
    for (int i = 0; i < N; ++i) x[i] = ldv_nt(ptrs.p[kMaxR + (int)((word >> (8 * i)) & 0xFF)] + off);
#pragma unroll
    for (int i = 0; i < N; ++i) slots[((int)((word >> (8 * i)) & 0xFF) * V + v) * T + tid] = x[i];
}

// The same fetch without staging registers: a 128-bit load that the memory pipeline writes
// straight into LDS (lane l of the wave lands at the wave-uniform LDS base + 16 l), so a thread
// can have every first-touch load of its program in flight at once.
__device__ __forceinline__ void slot_fetch_direct(const char* rank_base, u32x4* slots, int slot, int T, int tid, int64_t off) {
    const char* g = rank_base + off;
    u32x4* wave_base = slots + slot * T + (tid & ~63);
    __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)g,
                                     (__attribute__((address_space(3))) void*)wave_base, 16, 0, 2 /* nt */);
}

// A tile is T x V vectors of every rank: thread t owns vectors t, t + T, ..., t + (V - 1) T of it,
// so that every wave access is 1 KiB contiguous and the workgroup covers 16 T V contiguous bytes
// of each rank buffer.  What the memory system rewards (measured on MI355X with a bare kernel of
// this shape, 8 buffers of 512 MiB read and written in place): the same 32 KiB of slots as five
// workgroups of 256 threads per CU 5.97 TB/s; one workgroup per CU holding 64 KiB of slots, 8 KiB
// of every rank, 6.40 (256 threads x 2 vectors) to 6.55 TB/s (512 threads x 1); 128 KiB of slots
// 6.1 to 6.3.  Fewer, larger workgroups keep the requests of a CU in a narrow range of addresses.
// Elements [lo, hi) of a vector (0 <= lo <= hi <= elements per vector) to memory: the whole vector
// as one streaming store, a part of it element by element.
template <int DT>
__device__ __forceinline__ void store_vector_part(char* p, u32x4 x, int lo, int hi) {
    constexpr int ES = ElemBytes<DT>::value;
    constexpr int VE = 16 / ES;
    if (lo == 0 && hi == VE) { stv_nt(p, x); return; }
    for (int e = lo; e < hi; ++e) {
        const int wi = (e * ES) >> 2;
        const uint32_t word = wi == 0 ? x.x : wi == 1 ? x.y : wi == 2 ? x.z : x.w;
        store_elem<DT>(p + e * ES, word >> (((e * ES) & 3) * 8));
    }
}

// One tile of the slot runner.  MASKED: the tile is cut by the segment's ends.  Such a tile runs
// the same way with three differences: a vector that lies outside the segment is neither loaded nor
// stored; a vector that the boundary cuts is loaded whole - a 16-byte vector at a 16-byte boundary
// that holds one valid element lies in that element's page, so the load cannot fault, and what it
// brings in from beyond the boundary is computed on and thrown away - and stored element by
// element, only the elements inside.
template <int DT, bool DIRECT, int V, bool MASKED>
__device__ __forceinline__ void slot_tile(const ColumnLaunch& L, const DevColSegment& seg, const RankPtrs& ptrs,
                                          u32x4* slots, int64_t vfirst, int T, int tid) {
    constexpr int ES = ElemBytes<DT>::value;
    constexpr int VE = 16 / ES;
    const PCCL_CONST uint64_t* prog = as_const(L.instrs) + seg.prog_start;
    int64_t off[V];
    int elo[V], ehi[V];   // MASKED: the elements of vector v inside the segment
#pragma unroll
    for (int v = 0; v < V; ++v) {
        const int64_t vec = vfirst + (int64_t)v * T + tid;
        off[v] = vec * 16;
        elo[v] = 0; ehi[v] = VE;
        if constexpr (MASKED) {
            const int64_t e0 = vec * VE;
            const int64_t a = seg.start > e0 ? seg.start - e0 : 0, b = seg.end - e0 < VE ? seg.end - e0 : VE;
            elo[v] = (int)(a < VE ? a : VE);
            ehi[v] = (int)(b > elo[v] ? b : elo[v]);
        }
    }
    const PCCL_CONST uint64_t* pre = as_const(L.pre) + seg.pre_start;
    uint64_t w4[4] = {prog[0], prog[1], prog[2], prog[3]};
    if constexpr (DIRECT) {
        // the ranks this program reads by first touch, as a mask in the segment record: nothing
        // else has to be read before the first load can go out
        for (uint64_t m = seg.pre_mask; m; m &= m - 1) {
            const int rank = __builtin_ctzll(m);
            const char* base = ptrs.p[kMaxR + rank];
#pragma unroll
            for (int v = 0; v < V; ++v)
                if (!MASKED || ehi[v] > elo[v]) slot_fetch_direct(base, slots, rank * V + v, T, tid, off[v]);
        }
        // the loads above write LDS behind the compiler's back: wait for all of them before
        // any slot is read, and keep the slot reads below this point
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    } else {
        for (int i = 0; i < seg.pre_words; ++i) {
#pragma unroll
            for (int v = 0; v < V; ++v) {
                if (MASKED && ehi[v] <= elo[v]) continue;
                uint64_t word = pre[i];
                if ((word >> 56) != 0xFF) { slot_fetch<8>(word, ptrs, slots, V, v, T, tid, off[v]); continue; }
                if (((word >> 24) & 0xFF) != 0xFF) { slot_fetch<4>(word, ptrs, slots, V, v, T, tid, off[v]); word >>= 32; }
                if (((word >> 8) & 0xFF) != 0xFF) { slot_fetch<2>(word, ptrs, slots, V, v, T, tid, off[v]); word >>= 16; }
                if ((word & 0xFF) != 0xFF) slot_fetch<1>(word, ptrs, slots, V, v, T, tid, off[v]);
            }
        }
    }
    u32x4 acc[V];
#pragma unroll
    for (int v = 0; v < V; ++v) acc[v] = u32x4{0, 0, 0, 0};
    // The interpreter loop.  Programs are padded to a multiple of 4 instructions: one scalar load
    // brings in four (the first four were asked for before the wait above).  Forms of this loop
    // that read the next instruction's slot operands ahead, that read both operands
    // unconditionally to avoid branches, or that kept the rank pointers in lanes (v_readlane
    // instead of a scalar load per use) were measured and were no faster where several workgroups
    // share a CU, and slower for MAX programs; this plain form stays.
    for (int k = 0; k < seg.prog_len; k += 4) {
        if (k > 0) { w4[0] = prog[k]; w4[1] = prog[k + 1]; w4[2] = prog[k + 2]; w4[3] = prog[k + 3]; }
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const ColInstrDev in = unpack_instr(w4[j]);
            const u32x4* const pa = slots + (in.peer * V) * T + tid;
            u32x4* const ps = slots + (in.self * V) * T + tid;
            const int kind = in.store & 3;
            const bool to_mem = kind == 2 || (kind == 1 && (in.store & 4));
            char* const dst = ptrs.p[in.self];
#pragma unroll
            for (int v = 0; v < V; ++v) {
                const u32x4 a = in.a_src == 2 ? acc[v] : pa[v * T];
                if (in.b_src != 0) {
                    const u32x4 b = in.b_src == 2 ? acc[v] : ps[v * T];
                    acc[v] = vec_op<DT>(a, b, in.redop);
                } else acc[v] = a;
                if (kind == 1) ps[v * T] = acc[v];
                if (to_mem) {
                    if constexpr (MASKED) store_vector_part<DT>(dst + off[v], acc[v], elo[v], ehi[v]);
                    else stv_nt(dst + off[v], acc[v]);
                }
            }
        }
    }
    if constexpr (!MASKED) {
        if (L.slot_store_waves && seg.bcast_mask) {
            // The broadcast tail with the stores dealt to the waves: every thread parks its results in
            // its own rank-0 slots - slot (0, v) of thread t sits at index v T + t, so the parked
            // values lie in the order of the tile - and after a barrier wave w stores the whole tile
            // to the ranks of the mask that fall to it: 16 T V contiguous bytes of one rank from one
            // wave, instead of 1 KiB of every rank.  The host switches this on for plans that write at
            // least four times what they read in workgroups of four waves or more (an 8-rank 512 MB fp16
            // allgather 0.82 -> 0.79 ms); plans that read as much as they write are the same either
            // way, and two-wave workgroups get slower (32-rank tree 1.12 -> 1.28 ms).
#pragma unroll
            for (int v = 0; v < V; ++v) slots[v * T + tid] = acc[v];
            __syncthreads();
            const int W = T >> 6, w = tid >> 6, lane = tid & 63;
            int k = 0;
            for (uint64_t m = seg.bcast_mask; m; m &= m - 1, ++k) {
                if (k % W != w) continue;
                char* const dst = ptrs.p[__builtin_ctzll(m)] + vfirst * 16;
                for (int j = 0; j < T * V; j += 64) stv_nt(dst + (int64_t)(j + lane) * 16, slots[j + lane]);
            }
            __syncthreads();   // a workgroup that walks on to another tile fetches into these slots
            return;
        }
    }
    // the broadcast tail, four rank pointers fetched per round so that their scalar loads overlap
    for (uint64_t m = seg.bcast_mask; m;) {
        char* dsts[4];
        int n = 0;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int r = m ? __builtin_ctzll(m) : 0;
            if (m) { m &= m - 1; n = i + 1; }
            dsts[i] = ptrs.p[r];
        }
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            if (i >= n) break;
            char* const dst = dsts[i];
#pragma unroll
            for (int v = 0; v < V; ++v) {
                if constexpr (MASKED) store_vector_part<DT>(dst + off[v], acc[v], elo[v], ehi[v]);
                else stv_nt(dst + off[v], acc[v]);
            }
        }
    }
}

// (A workgroup has at most 1024 / V threads, so that the V-fold register need fits.)
template <int DT, bool DIRECT, int V>
__global__ __launch_bounds__(1024 / V) void column_slot_kernel(ColumnLaunch L, RankPtrs ptrs) {
    extern __shared__ u32x4 slots[];
    constexpr int ES = ElemBytes<DT>::value;
    constexpr int VE = 16 / ES;
    const int T = blockDim.x;
    const int tid = threadIdx.x;
    const int64_t tile_v = (int64_t)T * V;
    // A workgroup that walks several tiles (a grid capped at the number of workgroups resident at
    // once) keeps the segment record while its tiles stay in one segment: from the second tile on
    // nothing has to be read before the first load goes out.
    int have = -1;
    DevColSegment seg{};
    for (int64_t w = blockIdx.x; w < span_tiles(L.total_tiles, L.xcd_run); w += gridDim.x) {
        const int64_t tile = xcd_tile(w, L.xcd_run);
        if (tile >= L.total_tiles) continue;
        const int lo = find_segment(L, tile);
        if (lo != have) { seg = load_const(L.segs + lo); have = lo; }
        const int64_t vfirst = seg.first_vec + (tile - seg.first_tile) * tile_v;
        const bool interior = vfirst * VE >= seg.start && (vfirst + tile_v) * VE <= seg.end;
        if (interior) slot_tile<DT, DIRECT, V, false>(L, seg, ptrs, slots, vfirst, T, tid);
        else slot_tile<DT, DIRECT, V, true>(L, seg, ptrs, slots, vfirst, T, tid);
    }
}

// ------------------------------------------------------------------------------- phased runner
//
// Chain programs - one accumulator per position takes the ranks' original values one after another
// and the result goes to every rank of a mask: ring allreduce segments, staged reduce_scatter and
// allgather, trees under an operator that may be re-associated - run on a persistent grid of one
// workgroup per CU in which the WHOLE CHIP reads together and then writes together.  A workgroup
// takes a chunk of T x V vectors of every rank per sweep and keeps its V accumulators per thread in
// registers: read phase = every source rank's chunk streamed in through a small ring of LDS slots
// and combined; all workgroups meet; write phase = the accumulators stored to every rank of the
// mask; all meet again.  The memory system then sees long runs of pure reads and pure writes instead
// of a mix (measured on MI355X with bare kernels of this traffic shape, in place: 8 ranks x 512 MiB
// 67 % of the 8 TB/s peak without the meetings, 80 % with them, against 77 % for the best
// one-tile-per-workgroup shape; 32 ranks x 96 MiB 67 / 83 / 73 %).  The traffic is the same as the
// slot runner's: every rank read once, written once.
//
// The meetings order nothing - a workgroup only ever touches its own chunk - so they cannot make a
// result wrong, and they are bounded: a workgroup that waits longer than `timeout_ticks` (some
// workgroup is not resident, the GPU is shared) marks the launch as unsynchronised and everybody
// goes on without further waiting.  The last workgroup to leave clears the meeting block.
//
// Chunks that a segment boundary cuts are run vector by vector by the same workgroup (loads and
// stores of one vector together, cut vectors stored element by element): there are at most two per
// segment.
//
// Which vectors of its chunk a thread holds (LAY): 0 = the chunk as V slabs of T vectors, thread t
// vector t of every slab (all waves of a workgroup read and write one 1 KiB-per-wave slab together);
// 1 = each wave V KiB in a row, for reads and writes; 2 = read as slabs, written with each wave on
// V KiB in a row: the sums change hands through LDS between the two phases (T x V x 16 bytes, the
// fetch ring's space included).  Reads are fastest as slabs and writes with long runs per wave
// (bare kernels, 32 ranks x 96 MiB: read phases 6.9-7.0 against 6.8 TB/s, write phases 6.5 against
// 5.6-6.0); what the exchange costs is two LDS passes per sweep, about a microsecond in 80 to 330.

// One workgroup per CU: the kernel asks for more than half a CU's LDS, so that two cannot share one.
constexpr int kPhasedLdsBytes = 84 * 1024;

__device__ __forceinline__ void stv_nt_s(char* uniform_base, uint32_t off, u32x4 v) {
    asm volatile("global_store_dwordx4 %0, %1, %2 sc1 nt\n\ts_nop 0" : : "v"(off), "v"(v), "s"(uniform_base) : "memory");
}
__device__ __forceinline__ void load_lds_nt(const char* uniform_base, uint32_t off, u32x4* wave_base) {
    __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(uniform_base + off),
                                     (__attribute__((address_space(3))) void*)wave_base, 16, 0, 2 /* nt */);
}

__device__ __forceinline__ void phase_arrive(PhaseSync* s, int gen, int G) {
    if (threadIdx.x == 0) {
        const int old = __hip_atomic_fetch_add(&s->arrive, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if (old + 1 == gen * G) __hip_atomic_store(&s->release, gen, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
}
// Returns false once the launch is unsynchronised (this or another workgroup waited too long).
__device__ __forceinline__ bool phase_wait(PhaseSync* s, int gen, uint64_t timeout_ticks, int* s_flag) {
    if (threadIdx.x == 0) {
        int ok = 1;
        const uint64_t t0 = __builtin_amdgcn_s_memrealtime();
        while (__hip_atomic_load(&s->release, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) < gen) {
            if (__hip_atomic_load(&s->broken, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 0) { ok = 0; break; }
            if (__builtin_amdgcn_s_memrealtime() - t0 > timeout_ticks) {
                __hip_atomic_store(&s->broken, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                ok = 0;
                break;
            }
            __builtin_amdgcn_s_sleep(4);
        }
        *s_flag = ok;
    }
    __syncthreads();
    const int ok = __builtin_amdgcn_readfirstlane(*s_flag);
    __syncthreads();   // the flag may be rewritten by the next meeting
    return ok != 0;
}

// Read phase of one chunk: ranks srcs[0 .. n) streamed through a ring of S LDS slots per thread
// (S divides V, so the slot of vector v is v % S whatever the rank) and combined into acc[].
// Fetch q = k V + v is issued when fetch q - S has been consumed; loads complete in order, so
// "at most S - 1 outstanding" means fetch q has landed.
template <int DT, int OP, int T, int V, int S, int VS, int GR>
__device__ __forceinline__ void chain_read(u32x4 (&acc)[V], const PCCL_CONST int32_t* srcs, int n, const RankPtrs& ptrs,
                                           u32x4* lds, int64_t chunk_byte0, uint32_t toff, int tid) {
    static_assert(V % S == 0 && S <= V && S % GR == 0, "the slot of a vector must not depend on the rank; groups of GR vectors per wait");
    u32x4* const my = lds + (tid & ~63);
    const u32x4* const mine = lds + tid;
    const char* cur = ptrs.p[kMaxR + srcs[0]] + chunk_byte0;
#pragma unroll
    for (int q = 0; q < S; ++q) load_lds_nt(cur, toff + q * VS, my + q * T);
    for (int k = 0; k < n; ++k) {
        const bool last_rank = k + 1 == n;
        const char* next = ptrs.p[kMaxR + srcs[last_rank ? k : k + 1]] + chunk_byte0;
#pragma unroll
        for (int v = 0; v < V; v += GR) {
            // the GR oldest fetches have landed when at most S - GR are outstanding
            if (v + S >= V && last_rank) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            else asm volatile("s_waitcnt vmcnt(%0)" :: "n"(S - GR) : "memory");
            u32x4 x[GR];
#pragma unroll
            for (int g = 0; g < GR; ++g) x[g] = mine[((v + g) % S) * T];
#pragma unroll
            for (int g = 0; g < GR; ++g) acc[v + g] = k == 0 ? x[g] : vec_phase<DT, OP>(x[g], acc[v + g]);
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");   // the slots have been read before they are refilled
#pragma unroll
            for (int g = 0; g < GR; ++g) {
                const int w = v + g;
                if (w + S < V) load_lds_nt(cur, toff + (w + S) * VS, my + (w % S) * T);
                else if (!last_rank) load_lds_nt(next, toff + (w + S - V) * VS, my + (w % S) * T);
            }
        }
        cur = next;
    }
    if constexpr (kDeferredNan<DT>) {
        if (n > 1) {      // a single source is a copy: its bits are kept as they are
#pragma unroll
            for (int v = 0; v < V; ++v) acc[v] = canon_nan<DT>(acc[v]);
        }
    }
}

// The same for two chunks read in one phase (kept apart from chain_read, whose code the one-sweep
// kernels were tuned with: with these flags added there, the compiler scheduled the 32-rank f32 MAX
// kernel differently, 0.84 -> 0.79 of peak).  CIN: the ring already holds this chunk's first S
// fetches (the call before ended with COUT); COUT: the last rank's refills go on into `after`, the
// first source of the chunk read next, so that no fetch-free gap separates the two chunks.
template <int DT, int OP, int T, int V, int S, int VS, int GR, bool CIN, bool COUT>
__device__ __forceinline__ void chain_read_linked(u32x4 (&acc)[V], const PCCL_CONST int32_t* srcs, int n, const RankPtrs& ptrs,
                                           u32x4* lds, int64_t chunk_byte0, uint32_t toff, int tid, const char* after = nullptr) {
    static_assert(V % S == 0 && S <= V && S % GR == 0, "the slot of a vector must not depend on the rank; groups of GR vectors per wait");
    u32x4* const my = lds + (tid & ~63);
    const u32x4* const mine = lds + tid;
    const char* cur = ptrs.p[kMaxR + srcs[0]] + chunk_byte0;
    if constexpr (!CIN) {
#pragma unroll
        for (int q = 0; q < S; ++q) load_lds_nt(cur, toff + q * VS, my + q * T);
    }
    for (int k = 0; k < n; ++k) {
        const bool last_rank = k + 1 == n;
        const char* next = !last_rank ? ptrs.p[kMaxR + srcs[k + 1]] + chunk_byte0 : COUT ? after : cur;
#pragma unroll
        for (int v = 0; v < V; v += GR) {
            // the GR oldest fetches have landed when at most S - GR are outstanding
            if (!COUT && v + S >= V && last_rank) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            else asm volatile("s_waitcnt vmcnt(%0)" :: "n"(S - GR) : "memory");
            u32x4 x[GR];
#pragma unroll
            for (int g = 0; g < GR; ++g) x[g] = mine[((v + g) % S) * T];
#pragma unroll
            for (int g = 0; g < GR; ++g) acc[v + g] = k == 0 ? x[g] : vec_phase<DT, OP>(x[g], acc[v + g]);
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");   // the slots have been read before they are refilled
#pragma unroll
            for (int g = 0; g < GR; ++g) {
                const int w = v + g;
                if (w + S < V) load_lds_nt(cur, toff + (w + S) * VS, my + (w % S) * T);
                else if (COUT || !last_rank) load_lds_nt(next, toff + (w + S - V) * VS, my + (w % S) * T);
            }
        }
        cur = next;
    }
    if constexpr (kDeferredNan<DT>) {
        if (n > 1) {      // a single source is a copy: its bits are kept as they are
#pragma unroll
            for (int v = 0; v < V; ++v) acc[v] = canon_nan<DT>(acc[v]);
        }
    }
}

template <int V, class F, int... Vs>
__device__ __forceinline__ void fill_by_index(u32x4 (&out)[V], F&& f, std::integer_sequence<int, Vs...>) {
    ((out[Vs] = f(Vs)), ...);
}

// Read phase of one chunk whose value is a perfectly balanced tree over n = 2^depth ranks, depth >= 2:
// vector by vector, all n leaves of a vector before the next vector, four leaves at a time - a quad
// ((l0 + l1) + (l2 + l3)) is combined at once, and the quads' results climb the remaining levels like
// a binary counter over the quad number: quad j is combined with the parked left siblings of every
// level whose bit is set in j and is parked at the first level whose bit is clear.  The waiting left
// siblings are thus `depth - 2` vectors per thread whatever V is.  Fetch q = v n + k goes to slot
// q % S.  The leaves' base addresses sit in the lanes of one register pair (lane i: leaf i) and are
// picked with v_readlane: no memory access stands between two fetches.
template <int DT, int T, int V, int S, int VS>
__device__ __forceinline__ void tree_read(u32x4 (&acc)[V], const PCCL_CONST int32_t* srcs, int n, int depth, const RankPtrs& ptrs,
                                          u32x4* lds, int64_t chunk_byte0, uint32_t toff, int tid) {
    static_assert(S % 4 == 0 && S >= 8, "a quad is consumed while the next one is in flight");
    constexpr int kMaxUpper = 4;                 // levels above the quads: trees of up to 64 ranks
    u32x4* const my = lds + (tid & ~63);
    const u32x4* const mine = lds + tid;
    uint32_t lp_lo = 0, lp_hi = 0;
    for (int i = 0; i < n; ++i) {
        const uint64_t p = (uint64_t)(ptrs.p[kMaxR + srcs[i]] + chunk_byte0);
        if ((tid & 63) == i) { lp_lo = (uint32_t)p; lp_hi = (uint32_t)(p >> 32); }
    }
    auto leaf_base = [&](int k) {
        // (the builtin returns a signed int: without the casts a low word with its top bit set would
        // smear ones over the high word)
        const uint64_t p = (uint64_t)(uint32_t)__builtin_amdgcn_readlane((int)lp_lo, k) |
                           ((uint64_t)(uint32_t)__builtin_amdgcn_readlane((int)lp_hi, k) << 32);
        return (const char*)p;
    };
    const int total = V * n;                     // fetches of this chunk; total >= S because n >= 4 and V >= 2
    auto fetch = [&](int q) {                    // q uniform: leaf q % n of vector q / n into slot q % S
        load_lds_nt(leaf_base(q & (n - 1)), toff + (uint32_t)(q >> depth) * VS, my + (q & (S - 1)) * T);
    };
    for (int q = 0; q < S; ++q) fetch(q);
    const int upper = depth - 2;                 // levels the quads' results still have to climb
    u32x4 parked[kMaxUpper];
    // one vector: all its leaves, quad by quad; returns the root
    auto one_vector = [&](int v) __attribute__((always_inline)) {
        u32x4 root = u32x4{0, 0, 0, 0};
        for (int k = 0; k < n; k += 4) {
            const int q = v * n + k;
            if (q + S >= total) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            else asm volatile("s_waitcnt vmcnt(%0)" :: "n"(S - 4) : "memory");
            const u32x4 l0 = mine[(q & (S - 1)) * T], l1 = mine[((q + 1) & (S - 1)) * T];
            const u32x4 l2 = mine[((q + 2) & (S - 1)) * T], l3 = mine[((q + 3) & (S - 1)) * T];
            u32x4 y = vec_phase<DT, PCCL_SUM>(vec_phase<DT, PCCL_SUM>(l0, l1), vec_phase<DT, PCCL_SUM>(l2, l3));
            int climb = __builtin_ctz(~(unsigned)(k >> 2));      // trailing one bits of the quad number (uniform)
            if (climb > upper) climb = upper;
#pragma unroll
            for (int lvl = 0; lvl < kMaxUpper; ++lvl)
                if (lvl < climb) y = vec_phase<DT, PCCL_SUM>(parked[lvl], y);
#pragma unroll
            for (int lvl = 0; lvl < kMaxUpper; ++lvl)
                if (lvl == climb && lvl < upper) parked[lvl] = y;
            if (climb == upper) root = kDeferredNan<DT> ? canon_nan<DT>(y) : y;   // the last quad carries the root
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");   // the slots have been read before they are refilled
            if (q + S < total) { fetch(q + S); fetch(q + S + 1); fetch(q + S + 2); fetch(q + S + 3); }
        }
        return root;
    };
    // a fold over the vector numbers: every index of acc[] is a compile-time constant whatever the
    // optimiser makes of the loops inside
    fill_by_index(acc, one_vector, std::make_integer_sequence<int, V>{});
}

template <int DT, int T, int V, int S, int LAY, int GR, bool TREE>
__global__ __launch_bounds__(T) void phased_kernel(PhasedLaunch L, RankPtrs ptrs) {
    extern __shared__ u32x4 lds[];
    __shared__ int s_flag;
    static_assert((size_t)S * T * 16 <= 159u * 1024, "the fetch ring must fit a CU's LDS");
    static_assert(LAY != 2 || ((size_t)T * V * 16 <= 159u * 1024 && S <= V), "so must a chunk's sums when they change hands through it");
    constexpr int ES = ElemBytes<DT>::value;
    constexpr int VE = 16 / ES;
    constexpr int64_t CHUNK_V = (int64_t)T * V;
    constexpr int VS = LAY == 1 ? 64 * 16 : T * 16;          // bytes between a thread's consecutive vectors while it reads
    constexpr int WVS = LAY >= 1 ? 64 * 16 : T * 16;         // ... and while it writes
    const int tid = threadIdx.x;
    const int G = gridDim.x;
    // workgroup b runs on XCD b % 8: every XCD takes a contiguous eighth of each sweep
    const int place = (G & 7) == 0 ? (int)(blockIdx.x & 7) * (G >> 3) + (int)(blockIdx.x >> 3) : (int)blockIdx.x;
    // thread's first vector inside a chunk: each wave a contiguous V KiB, or the chunk as V slabs of T vectors
    const uint32_t wavec = (uint32_t)(tid >> 6) * V * 64 + (tid & 63);
    const uint32_t toff = (LAY == 1 ? wavec : (uint32_t)tid) * 16;
    const uint32_t wtoff = (LAY >= 1 ? wavec : (uint32_t)tid) * 16;
    const int64_t sweeps = (L.total_chunks + G - 1) / G;
    bool meet = L.barriers != 0;
    int gen = 0;
    for (int64_t it = 0; it < sweeps; ++it) {
        const int64_t chunk = it * G + place;
        const bool live = chunk < L.total_chunks;
        u32x4 acc[V];
#pragma unroll
        for (int v = 0; v < V; ++v) acc[v] = u32x4{0, 0, 0, 0};
        DevChainSegment seg{};
        int64_t vbase = 0;
        bool whole = false;
        if (live) {
            int lo = 0;
            if (L.seg_chunks > 0) {
                const uint32_t per = (uint32_t)L.seg_chunks;
                lo = (per & (per - 1)) == 0 ? (int)((uint32_t)chunk >> __builtin_ctz(per)) : (int)((uint32_t)chunk / per);
            } else {
                int hi = L.num_segs;
                while (hi - lo > 1) {
                    const int mid = (lo + hi) >> 1;
                    if (as_const(L.segs)[mid].first_chunk <= chunk) lo = mid; else hi = mid;
                }
            }
            seg = load_const(L.segs + lo);
            vbase = seg.first_vec + (chunk - seg.first_chunk) * CHUNK_V;
            whole = vbase * VE >= seg.start && (vbase + CHUNK_V) * VE <= seg.end;
            const PCCL_CONST int32_t* srcs = as_const(L.srcs) + seg.src_start;   // dwords: uniform reads become scalar loads
            if (whole) {
                bool done = false;
                if constexpr (TREE) {
                    if (seg.tree_depth > 1) { tree_read<DT, T, V, S, VS>(acc, srcs, seg.n_src, seg.tree_depth, ptrs, lds, vbase * 16, toff, tid); done = true; }
                }
                if (done) {}
                else if (seg.redop == PCCL_SUM) chain_read<DT, PCCL_SUM, T, V, S, VS, GR>(acc, srcs, seg.n_src, ptrs, lds, vbase * 16, toff, tid);
                else if (seg.redop == PCCL_MAX) chain_read<DT, PCCL_MAX, T, V, S, VS, GR>(acc, srcs, seg.n_src, ptrs, lds, vbase * 16, toff, tid);
                else chain_read<DT, PCCL_MIN, T, V, S, VS, GR>(acc, srcs, seg.n_src, ptrs, lds, vbase * 16, toff, tid);
            } else {
                // a chunk that the segment's ends cut: vector by vector, loads and stores together
                for (int64_t j = tid; j < CHUNK_V; j += T) {
                    const int64_t vec = vbase + j;
                    int64_t e0 = vec * VE, e1 = e0 + VE;
                    if (e0 < seg.start) e0 = seg.start;
                    if (e1 > seg.end) e1 = seg.end;
                    if (e0 >= e1) continue;
                    u32x4 x = ldv(ptrs.p[kMaxR + srcs[0]] + vec * 16);
                    if (!TREE || seg.tree_depth == 0) {
                        for (int k = 1; k < seg.n_src; ++k) x = vec_op<DT>(ldv(ptrs.p[kMaxR + srcs[k]] + vec * 16), x, seg.redop);
                    } else {
                        u32x4 parked[6];
                        for (int k = 0; k < seg.n_src; ++k) {
                            u32x4 y = k == 0 ? x : ldv(ptrs.p[kMaxR + srcs[k]] + vec * 16);
                            bool placed = false;
#pragma unroll
                            for (int lvl = 0; lvl < 6; ++lvl) {
                                if (!placed && lvl < seg.tree_depth) {
                                    if (k >> lvl & 1) y = vec_op<DT>(parked[lvl], y, seg.redop);
                                    else { parked[lvl] = y; placed = true; }
                                }
                            }
                            if (!placed) x = y;
                        }
                    }
                    for (uint64_t m = seg.store_mask; m; m &= m - 1)
                        store_vector_part<DT>(ptrs.p[__builtin_ctzll(m)] + vec * 16, x, (int)(e0 - vec * VE), (int)(e1 - vec * VE));
                }
            }
        }
        if constexpr (LAY == 2) {
            if (live && whole) {            // uniform over the workgroup: the barriers are reached by all or by none
                asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
                __syncthreads();            // every wave has consumed its ring slots: the space is free
#pragma unroll
                for (int v = 0; v < V; ++v) lds[v * T + tid] = acc[v];          // position v T + t of the chunk
                __syncthreads();
#pragma unroll
                for (int v = 0; v < V; ++v) acc[v] = lds[wavec + v * 64];
                asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
                __syncthreads();            // all have their sums before the next sweep's fetches land here
            }
        }
        if (meet) {
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            __syncthreads();
            ++gen;
            phase_arrive(L.sync, gen, G);
            meet = phase_wait(L.sync, gen, L.timeout_ticks, &s_flag);
        }
        if (live && whole) {
            for (uint64_t m = seg.store_mask; m; m &= m - 1) {
                char* const dst = ptrs.p[__builtin_ctzll(m)] + vbase * 16;
#pragma unroll
                for (int v = 0; v < V; ++v) stv_nt_s(dst, wtoff + v * WVS, acc[v]);
            }
        }
        if (meet && it + 1 < sweeps) {
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            __syncthreads();
            ++gen;
            phase_arrive(L.sync, gen, G);
            meet = phase_wait(L.sync, gen, L.timeout_ticks, &s_flag);
        }
    }
    // the last workgroup to leave clears the meeting block for the next launch
    if (L.barriers != 0 && tid == 0) {
        const int old = __hip_atomic_fetch_add(&L.sync->exited, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if (old + 1 == G) {
            __hip_atomic_store(&L.sync->arrive, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            __hip_atomic_store(&L.sync->release, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            __hip_atomic_store(&L.sync->broken, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            __hip_atomic_store(&L.sync->exited, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
    }
}

// The same runner with KK sweeps read before their sums are written: the phases are KK times as long
// and the meetings KK times fewer.  Worth most for plans that store little (a reduce_scatter: R
// chunks in, one out), where a write phase per sweep would be too short to be worth a meeting and
// without meetings the stores sprinkle the reads (bare kernels of this traffic, 8 x 512 MiB in and
// 8 x 64 MiB out: 0.788 of peak without meetings, 0.804 with a write phase per sweep, 0.865 per two
// sweeps, 0.868 per three); an allreduce in place on 8 ranks gains one to two points.  Two whole
// chunks are read as ONE fetch stream: the ring runs on from the last rank of the first chunk into
// the first rank of the second, so no fetch-free gap (one memory latency, chip-wide) separates them;
// without that the f32 and f16 forms, whose NaN pass sits in that gap, lost what the longer phases
// gained.  Chains read and written as slabs only; a kernel of its own, so that the one above keeps
// the code it was tuned with.
template <int DT, int T, int V, int S, int GR, int KK>
__global__ __launch_bounds__(T) void phased_kernel_pairs(PhasedLaunch L, RankPtrs ptrs) {
    extern __shared__ u32x4 lds[];
    __shared__ int s_flag;
    static_assert((size_t)S * T * 16 <= 159u * 1024, "the fetch ring must fit a CU's LDS");
    static_assert(KK >= 1 && KK <= 2 && KK * V <= 32, "the sums of KK sweeps stay in registers; one call of read_sweep per sweep below");
    constexpr int ES = ElemBytes<DT>::value;
    constexpr int VE = 16 / ES;
    constexpr int64_t CHUNK_V = (int64_t)T * V;
    constexpr int VS = T * 16;                   // bytes between a thread's consecutive vectors: the chunk as V slabs
    const int tid = threadIdx.x;
    const int G = gridDim.x;
    // workgroup b runs on XCD b % 8: every XCD takes a contiguous eighth of each sweep
    const int place = (G & 7) == 0 ? (int)(blockIdx.x & 7) * (G >> 3) + (int)(blockIdx.x >> 3) : (int)blockIdx.x;
    const uint32_t toff = (uint32_t)tid * 16;
    const int64_t sweeps = (L.total_chunks + G - 1) / G;
    bool meet = L.barriers != 0;
    int gen = 0;
    for (int64_t it0 = 0; it0 < sweeps; it0 += KK) {
        u32x4 acc[KK][V];
        DevChainSegment seg[KK];
        int64_t vbase[KK];
        bool whole[KK];
        // (generic lambdas called once per constant k: the compiler does not unroll a loop with these bodies,
        // and with k a variable the per-sweep state would not stay in scalar registers)
        auto find_sweep = [&](auto kc) __attribute__((always_inline)) {
            constexpr int k = decltype(kc)::value;
            const int64_t chunk = (it0 + k) * G + place;
            const bool live = it0 + k < sweeps && chunk < L.total_chunks;
#pragma unroll
            for (int v = 0; v < V; ++v) acc[k][v] = u32x4{0, 0, 0, 0};
            seg[k] = DevChainSegment{};
            vbase[k] = 0;
            whole[k] = false;
            if (!live) return false;
            int lo = 0;
            if (L.seg_chunks > 0) {
                const uint32_t per = (uint32_t)L.seg_chunks;
                lo = (per & (per - 1)) == 0 ? (int)((uint32_t)chunk >> __builtin_ctz(per)) : (int)((uint32_t)chunk / per);
            } else {
                int hi = L.num_segs;
                while (hi - lo > 1) {
                    const int mid = (lo + hi) >> 1;
                    if (as_const(L.segs)[mid].first_chunk <= chunk) lo = mid; else hi = mid;
                }
            }
            seg[k] = load_const(L.segs + lo);
            vbase[k] = seg[k].first_vec + (chunk - seg[k].first_chunk) * CHUNK_V;
            whole[k] = vbase[k] * VE >= seg[k].start && (vbase[k] + CHUNK_V) * VE <= seg[k].end;
            return true;
        };
        // CIN / COUT: the fetch ring runs on from this sweep's chunk into the next one's (chain_read_linked)
        auto read_sweep = [&](auto kc, auto cin, auto cout, const char* after) __attribute__((always_inline)) {
            constexpr int k = decltype(kc)::value;
            constexpr bool CIN = decltype(cin)::value, COUT = decltype(cout)::value;
            const PCCL_CONST int32_t* srcs = as_const(L.srcs) + seg[k].src_start;   // dwords: uniform reads become scalar loads
            if (whole[k]) {
                if (seg[k].redop == PCCL_SUM) chain_read_linked<DT, PCCL_SUM, T, V, S, VS, GR, CIN, COUT>(acc[k], srcs, seg[k].n_src, ptrs, lds, vbase[k] * 16, toff, tid, after);
                else if (seg[k].redop == PCCL_MAX) chain_read_linked<DT, PCCL_MAX, T, V, S, VS, GR, CIN, COUT>(acc[k], srcs, seg[k].n_src, ptrs, lds, vbase[k] * 16, toff, tid, after);
                else chain_read_linked<DT, PCCL_MIN, T, V, S, VS, GR, CIN, COUT>(acc[k], srcs, seg[k].n_src, ptrs, lds, vbase[k] * 16, toff, tid, after);
            } else {
                // a chunk that the segment's ends cut: vector by vector, loads and stores together
                for (int64_t j = tid; j < CHUNK_V; j += T) {
                    const int64_t vec = vbase[k] + j;
                    int64_t e0 = vec * VE, e1 = e0 + VE;
                    if (e0 < seg[k].start) e0 = seg[k].start;
                    if (e1 > seg[k].end) e1 = seg[k].end;
                    if (e0 >= e1) continue;
                    u32x4 x = ldv(ptrs.p[kMaxR + srcs[0]] + vec * 16);
                    for (int i = 1; i < seg[k].n_src; ++i) x = vec_op<DT>(ldv(ptrs.p[kMaxR + srcs[i]] + vec * 16), x, seg[k].redop);
                    for (uint64_t m = seg[k].store_mask; m; m &= m - 1)
                        store_vector_part<DT>(ptrs.p[__builtin_ctzll(m)] + vec * 16, x, (int)(e0 - vec * VE), (int)(e1 - vec * VE));
                }
            }
        };
        constexpr std::integral_constant<int, 0> k0{};
        constexpr std::integral_constant<int, 1> k1{};
        constexpr std::false_type no{};
        constexpr std::true_type yes{};
        const bool live0 = find_sweep(k0);
        bool live1 = false;
        if constexpr (KK > 1) live1 = find_sweep(k1);
        if (KK > 1 && whole[0] && whole[KK - 1]) {
            // both chunks whole: one fetch stream through both
            const char* after = ptrs.p[kMaxR + as_const(L.srcs)[seg[KK - 1].src_start]] + vbase[KK - 1] * 16;
            read_sweep(k0, no, yes, after);
            if constexpr (KK > 1) read_sweep(k1, yes, no, nullptr);
        } else {
            if (live0) read_sweep(k0, no, no, nullptr);
            if constexpr (KK > 1) { if (live1) read_sweep(k1, no, no, nullptr); }
        }
        if (meet) {
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            __syncthreads();
            ++gen;
            phase_arrive(L.sync, gen, G);
            meet = phase_wait(L.sync, gen, L.timeout_ticks, &s_flag);
        }
        auto write_sweep = [&](auto kc) __attribute__((always_inline)) {
            constexpr int k = decltype(kc)::value;
            if (whole[k]) {
                for (uint64_t m = seg[k].store_mask; m; m &= m - 1) {
                    char* const dst = ptrs.p[__builtin_ctzll(m)] + vbase[k] * 16;
#pragma unroll
                    for (int v = 0; v < V; ++v) stv_nt_s(dst, toff + v * VS, acc[k][v]);
                }
            }
        };
        write_sweep(std::integral_constant<int, 0>{});
        if constexpr (KK > 1) write_sweep(std::integral_constant<int, 1>{});
        if (meet && it0 + KK < sweeps) {
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            __syncthreads();
            ++gen;
            phase_arrive(L.sync, gen, G);
            meet = phase_wait(L.sync, gen, L.timeout_ticks, &s_flag);
        }
    }
    // the last workgroup to leave clears the meeting block for the next launch
    if (L.barriers != 0 && tid == 0) {
        const int old = __hip_atomic_fetch_add(&L.sync->exited, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if (old + 1 == G) {
            __hip_atomic_store(&L.sync->arrive, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            __hip_atomic_store(&L.sync->release, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            __hip_atomic_store(&L.sync->broken, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            __hip_atomic_store(&L.sync->exited, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
    }
}

// The 256 x 32 shape with the chunks of K neighbouring workgroups INTERLEAVED slab by slab: the K
// chunks of a group are consecutive chunks of one segment, and slab v of workgroup j of the group is
// piece (v K + j) of that region, T vectors long.  At every step of a phase the group then reads or
// writes K x 4 KiB in a row - with K = 128 or 256 the chip sweeps each rank buffer as one linear
// stream 0.5 to 1 MiB wide instead of 256 separate streams 128 KiB apart.  Bare kernels, 8 ranks x
// 512 MiB in place: 0.824-0.828 of the 8 TB/s against 0.776 for the same shape with a chunk per
// workgroup and 0.802-0.806 for 512 x 16 (write phases 6.5-6.6 TB/s against 5.8 and 6.0-6.1); groups
// of 64 give 0.81, of 32 and fewer nothing.  At 16 and 32 ranks the shape that writes 32 KiB runs per
// wave stays ahead.  Chains only, every chunk whole (the host checks), one sweep per write phase.
template <int DT, int OP, int T, int V, int S, int GR>
__device__ __forceinline__ void chain_read_strided(u32x4 (&acc)[V], const PCCL_CONST int32_t* srcs, int n, const RankPtrs& ptrs,
                                                   u32x4* lds, int64_t first_byte, uint32_t toff, uint32_t vs, int tid) {
    static_assert(V % S == 0 && S <= V && S % GR == 0, "the slot of a vector must not depend on the rank; groups of GR vectors per wait");
    u32x4* const my = lds + (tid & ~63);
    const u32x4* const mine = lds + tid;
    const char* cur = ptrs.p[kMaxR + srcs[0]] + first_byte;
#pragma unroll
    for (int q = 0; q < S; ++q) load_lds_nt(cur, toff + q * vs, my + q * T);
    for (int k = 0; k < n; ++k) {
        const bool last_rank = k + 1 == n;
        const char* next = ptrs.p[kMaxR + srcs[last_rank ? k : k + 1]] + first_byte;
#pragma unroll
        for (int v = 0; v < V; v += GR) {
            if (v + S >= V && last_rank) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            else asm volatile("s_waitcnt vmcnt(%0)" :: "n"(S - GR) : "memory");
            u32x4 x[GR];
#pragma unroll
            for (int g = 0; g < GR; ++g) x[g] = mine[((v + g) % S) * T];
#pragma unroll
            for (int g = 0; g < GR; ++g) acc[v + g] = k == 0 ? x[g] : vec_phase<DT, OP>(x[g], acc[v + g]);
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");   // the slots have been read before they are refilled
#pragma unroll
            for (int g = 0; g < GR; ++g) {
                const int w = v + g;
                if (w + S < V) load_lds_nt(cur, toff + (w + S) * vs, my + (w % S) * T);
                else if (!last_rank) load_lds_nt(next, toff + (w + S - V) * vs, my + (w % S) * T);
            }
        }
        cur = next;
    }
    if constexpr (kDeferredNan<DT>) {
        if (n > 1) {
#pragma unroll
            for (int v = 0; v < V; ++v) acc[v] = canon_nan<DT>(acc[v]);
        }
    }
}

template <int DT, int T, int V, int S, int GR>
__global__ __launch_bounds__(T) void phased_kernel_linear(PhasedLaunch L, RankPtrs ptrs) {
    extern __shared__ u32x4 lds[];
    __shared__ int s_flag;
    static_assert((size_t)S * T * 16 <= 159u * 1024, "the fetch ring must fit a CU's LDS");
    constexpr int64_t CHUNK_V = (int64_t)T * V;
    const int tid = threadIdx.x;
    const int G = gridDim.x;
    const int K = L.group;                               // a power of two that divides G and every segment's chunk count
    const int kshift = __builtin_ctz((unsigned)K);
    // workgroup b runs on XCD b % 8: every XCD takes a contiguous eighth of each sweep
    const int place = (G & 7) == 0 ? (int)(blockIdx.x & 7) * (G >> 3) + (int)(blockIdx.x >> 3) : (int)blockIdx.x;
    const uint32_t toff = (uint32_t)tid * 16;
    const uint32_t vs = (uint32_t)K * T * 16;            // bytes between a thread's consecutive vectors
    const int64_t sweeps = (L.total_chunks + G - 1) / G;
    bool meet = L.barriers != 0;
    int gen = 0;
    for (int64_t it = 0; it < sweeps; ++it) {
        const int64_t chunk = it * G + place;
        const bool live = chunk < L.total_chunks;
        u32x4 acc[V];
#pragma unroll
        for (int v = 0; v < V; ++v) acc[v] = u32x4{0, 0, 0, 0};
        DevChainSegment seg{};
        int64_t first_byte = 0;
        if (live) {
            int lo = 0;
            if (L.seg_chunks > 0) {
                const uint32_t per = (uint32_t)L.seg_chunks;
                lo = (per & (per - 1)) == 0 ? (int)((uint32_t)chunk >> __builtin_ctz(per)) : (int)((uint32_t)chunk / per);
            } else {
                int hi = L.num_segs;
                while (hi - lo > 1) {
                    const int mid = (lo + hi) >> 1;
                    if (as_const(L.segs)[mid].first_chunk <= chunk) lo = mid; else hi = mid;
                }
            }
            seg = load_const(L.segs + lo);
            const int64_t rel = chunk - seg.first_chunk;            // the chunk's number inside its segment
            const int64_t first_vec = seg.first_vec + ((rel >> kshift) << kshift) * CHUNK_V + (rel & (K - 1)) * T;
            first_byte = first_vec * 16;
            const PCCL_CONST int32_t* srcs = as_const(L.srcs) + seg.src_start;   // dwords: uniform reads become scalar loads
            if (seg.redop == PCCL_SUM) chain_read_strided<DT, PCCL_SUM, T, V, S, GR>(acc, srcs, seg.n_src, ptrs, lds, first_byte, toff, vs, tid);
            else if (seg.redop == PCCL_MAX) chain_read_strided<DT, PCCL_MAX, T, V, S, GR>(acc, srcs, seg.n_src, ptrs, lds, first_byte, toff, vs, tid);
            else chain_read_strided<DT, PCCL_MIN, T, V, S, GR>(acc, srcs, seg.n_src, ptrs, lds, first_byte, toff, vs, tid);
        }
        if (meet) {
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            __syncthreads();
            ++gen;
            phase_arrive(L.sync, gen, G);
            meet = phase_wait(L.sync, gen, L.timeout_ticks, &s_flag);
        }
        if (live) {
            for (uint64_t m = seg.store_mask; m; m &= m - 1) {
                char* const dst = ptrs.p[__builtin_ctzll(m)] + first_byte;
#pragma unroll
                for (int v = 0; v < V; ++v) stv_nt_s(dst, toff + v * vs, acc[v]);
            }
        }
        if (meet && it + 1 < sweeps) {
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            __syncthreads();
            ++gen;
            phase_arrive(L.sync, gen, G);
            meet = phase_wait(L.sync, gen, L.timeout_ticks, &s_flag);
        }
    }
    // the last workgroup to leave clears the meeting block for the next launch
    if (L.barriers != 0 && tid == 0) {
        const int old = __hip_atomic_fetch_add(&L.sync->exited, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if (old + 1 == G) {
            __hip_atomic_store(&L.sync->arrive, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            __hip_atomic_store(&L.sync->release, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            __hip_atomic_store(&L.sync->broken, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            __hip_atomic_store(&L.sync->exited, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
    }
}

// The interleaved shape for segments SHORTER than a group: a group of K workgroups spans NS adjacent
// segments of K / NS chunks.  The group's region is V rows of K x T vectors; row v lies in segment
// v / (V / NS) of the group, so the slabs of a thread belong to different segments and are combined in
// different source orders: at step k of the chain, row v is fetched from the k-th source of ITS
// segment.  The host has checked that the segments of the plan are adjacent in memory and have the
// same number of sources, operator and store mask, their source lists one after the other.
template <int DT, int OP, int T, int V, int S, int GR, int NS>
__device__ __forceinline__ void chain_read_rows(u32x4 (&acc)[V], const PCCL_CONST int32_t* srcs0, int n, const RankPtrs& ptrs,
                                                u32x4* lds, int64_t first_byte, uint32_t toff, uint32_t vs, int tid) {
    static_assert(V % S == 0 && S <= V && S % GR == 0 && V % NS == 0, "slots must not depend on the rank; whole rows per segment");
    constexpr int RP = V / NS;                   // rows per segment
    u32x4* const my = lds + (tid & ~63);
    const u32x4* const mine = lds + tid;
    const char* pc[NS];
    const char* pn[NS];
#pragma unroll
    for (int si = 0; si < NS; ++si) pc[si] = ptrs.p[kMaxR + srcs0[si * n]] + first_byte;
#pragma unroll
    for (int q = 0; q < S; ++q) load_lds_nt(pc[q / RP], toff + q * vs, my + q * T);
    for (int k = 0; k < n; ++k) {
        const bool last_rank = k + 1 == n;
#pragma unroll
        for (int si = 0; si < NS; ++si) pn[si] = last_rank ? pc[si] : ptrs.p[kMaxR + srcs0[si * n + k + 1]] + first_byte;
#pragma unroll
        for (int v = 0; v < V; v += GR) {
            if (v + S >= V && last_rank) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            else asm volatile("s_waitcnt vmcnt(%0)" :: "n"(S - GR) : "memory");
            u32x4 x[GR];
#pragma unroll
            for (int g = 0; g < GR; ++g) x[g] = mine[((v + g) % S) * T];
#pragma unroll
            for (int g = 0; g < GR; ++g) acc[v + g] = k == 0 ? x[g] : vec_phase<DT, OP>(x[g], acc[v + g]);
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");   // the slots have been read before they are refilled
#pragma unroll
            for (int g = 0; g < GR; ++g) {
                const int w = v + g;
                if (w + S < V) load_lds_nt(pc[(w + S) / RP], toff + (w + S) * vs, my + (w % S) * T);
                else if (!last_rank) load_lds_nt(pn[(w + S - V) / RP], toff + (w + S - V) * vs, my + (w % S) * T);
            }
        }
#pragma unroll
        for (int si = 0; si < NS; ++si) pc[si] = pn[si];
    }
    if constexpr (kDeferredNan<DT>) {
        if (n > 1) {
#pragma unroll
            for (int v = 0; v < V; ++v) acc[v] = canon_nan<DT>(acc[v]);
        }
    }
}

template <int DT, int T, int V, int S, int GR, int NS>
__global__ __launch_bounds__(T) void phased_kernel_linear_rows(PhasedLaunch L, RankPtrs ptrs) {
    extern __shared__ u32x4 lds[];
    __shared__ int s_flag;
    static_assert((size_t)S * T * 16 <= 159u * 1024, "the fetch ring must fit a CU's LDS");
    const int tid = threadIdx.x;
    const int G = gridDim.x;
    const int K = L.group;                               // a power of two that divides G; NS segments of K / NS chunks per group
    const int kshift = __builtin_ctz((unsigned)K);
    const int place = (G & 7) == 0 ? (int)(blockIdx.x & 7) * (G >> 3) + (int)(blockIdx.x >> 3) : (int)blockIdx.x;
    const uint32_t toff = (uint32_t)tid * 16;
    const uint32_t vs = (uint32_t)K * T * 16;
    const int64_t sweeps = (L.total_chunks + G - 1) / G;
    bool meet = L.barriers != 0;
    int gen = 0;
    for (int64_t it = 0; it < sweeps; ++it) {
        const int64_t chunk = it * G + place;
        const bool live = chunk < L.total_chunks;
        u32x4 acc[V];
#pragma unroll
        for (int v = 0; v < V; ++v) acc[v] = u32x4{0, 0, 0, 0};
        DevChainSegment seg{};
        int64_t first_byte = 0;
        if (live) {
            const int64_t group = chunk >> kshift;
            seg = load_const(L.segs + group * NS);          // the group's first segment; the others follow it in memory
            first_byte = (seg.first_vec + (chunk & (K - 1)) * T) * 16;
            const PCCL_CONST int32_t* srcs0 = as_const(L.srcs) + seg.src_start;
            if (seg.redop == PCCL_SUM) chain_read_rows<DT, PCCL_SUM, T, V, S, GR, NS>(acc, srcs0, seg.n_src, ptrs, lds, first_byte, toff, vs, tid);
            else if (seg.redop == PCCL_MAX) chain_read_rows<DT, PCCL_MAX, T, V, S, GR, NS>(acc, srcs0, seg.n_src, ptrs, lds, first_byte, toff, vs, tid);
            else chain_read_rows<DT, PCCL_MIN, T, V, S, GR, NS>(acc, srcs0, seg.n_src, ptrs, lds, first_byte, toff, vs, tid);
        }
        if (meet) {
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            __syncthreads();
            ++gen;
            phase_arrive(L.sync, gen, G);
            meet = phase_wait(L.sync, gen, L.timeout_ticks, &s_flag);
        }
        if (live) {
            for (uint64_t m = seg.store_mask; m; m &= m - 1) {
                char* const dst = ptrs.p[__builtin_ctzll(m)] + first_byte;
#pragma unroll
                for (int v = 0; v < V; ++v) stv_nt_s(dst, toff + v * vs, acc[v]);
            }
        }
        if (meet && it + 1 < sweeps) {
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            __syncthreads();
            ++gen;
            phase_arrive(L.sync, gen, G);
            meet = phase_wait(L.sync, gen, L.timeout_ticks, &s_flag);
        }
    }
    if (L.barriers != 0 && tid == 0) {
        const int old = __hip_atomic_fetch_add(&L.sync->exited, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if (old + 1 == G) {
            __hip_atomic_store(&L.sync->arrive, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            __hip_atomic_store(&L.sync->release, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            __hip_atomic_store(&L.sync->broken, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            __hip_atomic_store(&L.sync->exited, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
    }
}

// ------------------------------------------------------------------------------- launchers

// Per-device facts, queried once.  Contexts on different threads may ask at the same time: the
// slots are atomics and every thread that finds one empty computes the same value.
constexpr int kMaxDevices = 16;
static std::atomic<int> g_cu_count[kMaxDevices];

static int current_device() {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) dev = 0;
    return dev;
}

int device_cu_count(int device) {
    if (device < 0 || device >= kMaxDevices) device = 0;
    int n = g_cu_count[device].load(std::memory_order_relaxed);
    if (!n) {
        if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, device) != hipSuccess || n <= 0) n = 256;
        g_cu_count[device].store(n, std::memory_order_relaxed);
    }
    return n;
}

static int current_cus() { return device_cu_count(current_device()); }

// Run length of the tile-to-XCD mapping for a launch over `ntiles` tiles: kXcdRun, halved while the
// launch is too small to give every XCD a whole run (small launches then start no idle workgroups).
static int run_for_tiles(int64_t ntiles) {
    int run = kXcdRun;
    while (run > 1 && (int64_t)kXcds * run > ntiles) run >>= 1;
    return run;
}

static int grid_for_tiles(int64_t ntiles, int run) {
    const int64_t cap = 1 << 30;   // the kernels stride over the tiles if a range ever exceeds this
    ntiles = span_tiles(ntiles > 0 ? ntiles : 1, run);
    return (int)(ntiles < cap ? ntiles : cap);
}

// The slot runner's launch: L.slot_vecs vectors per thread, L.slot_lds_bytes of dynamic LDS (at
// least the slots; more to limit the workgroups per CU).  More than 64 KiB of dynamic LDS has to be
// allowed per kernel and device once.
template <class K>
static int launch_slot_kernel(K kernel, std::atomic<int>* allowed, const ColumnLaunch& L, const RankPtrs& ptrs, unsigned grid, hipStream_t s) {
    const int dev = current_device();
    const int lds = L.slot_lds_bytes;
    if (L.slot_threads * L.slot_vecs > 1024) return (int)hipErrorInvalidValue;   // the kernels' launch bounds
    if (lds > 64 * 1024 && allowed[dev].load(std::memory_order_relaxed) < lds) {
        hipError_t rc = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, lds);
        if (rc != hipSuccess) return (int)rc;
        allowed[dev].store(lds, std::memory_order_relaxed);
    }
    hipLaunchKernelGGL(kernel, dim3(grid), dim3(L.slot_threads), (size_t)lds, s, L, ptrs);
    return (int)hipGetLastError();
}

template <int DT>
static int launch_slot_dt(const ColumnLaunch& L, const RankPtrs& ptrs, unsigned grid, hipStream_t s) {
    static std::atomic<int> allowed[5][kMaxDevices];   // per kernel of this element type
    if (L.slot_direct) {
        switch (L.slot_vecs) {
            case 1: return launch_slot_kernel(column_slot_kernel<DT, true, 1>, allowed[0], L, ptrs, grid, s);
            case 2: return launch_slot_kernel(column_slot_kernel<DT, true, 2>, allowed[1], L, ptrs, grid, s);
            case 4: return launch_slot_kernel(column_slot_kernel<DT, true, 4>, allowed[2], L, ptrs, grid, s);
            default: return (int)hipErrorInvalidValue;
        }
    }
    if (L.slot_vecs != 1) return (int)hipErrorInvalidValue;   // fetching through registers: one vector per thread
    return launch_slot_kernel(column_slot_kernel<DT, false, 1>, allowed[3], L, ptrs, grid, s);
}

template <int DT>
static int launch_column_dt(const ColumnLaunch& L0, const RankPtrs& ptrs, hipStream_t s) {
    ColumnLaunch L = L0;
    L.xcd_run = run_for_tiles(L.total_tiles);
    int64_t grid = span_tiles(L.total_tiles, L.xcd_run);
    if (L.num_blocks > 0 && grid > L.num_blocks) grid = L.num_blocks;
    if (grid > (1 << 30)) grid = 1 << 30;
    if (grid <= 0) return 0;
    if (L.slot_threads > 0) return launch_slot_dt<DT>(L, ptrs, (unsigned)grid, s);
    switch (L.vecs_per_thread) {
        case 1: hipLaunchKernelGGL((column_kernel<DT, 1>), dim3((unsigned)grid), dim3(kThreads), 0, s, L, ptrs); break;
        case 2: hipLaunchKernelGGL((column_kernel<DT, 2>), dim3((unsigned)grid), dim3(kThreads), 0, s, L, ptrs); break;
        default: hipLaunchKernelGGL((column_kernel<DT, 4>), dim3((unsigned)grid), dim3(kThreads), 0, s, L, ptrs); break;
    }
    return (int)hipGetLastError();
}

int launch_column(const ColumnLaunch& L, const RankPtrs& ptrs, void* stream) {
    hipStream_t s = (hipStream_t)stream;
    switch (L.dtype) {
        case PCCL_F32: return launch_column_dt<PCCL_F32>(L, ptrs, s);
        case PCCL_F16: return launch_column_dt<PCCL_F16>(L, ptrs, s);
        case PCCL_BF16: return launch_column_dt<PCCL_BF16>(L, ptrs, s);
        case PCCL_I32: return launch_column_dt<PCCL_I32>(L, ptrs, s);
        case PCCL_F8E4M3: return launch_column_dt<PCCL_F8E4M3>(L, ptrs, s);
        case PCCL_F8E5M2: return launch_column_dt<PCCL_F8E5M2>(L, ptrs, s);
        default: return (int)hipErrorInvalidValue;
    }
}

template <class K>
static int launch_phased_kernel(K kernel, std::atomic<int>* allowed, int threads, int lds_vectors, const PhasedLaunch& L, const RankPtrs& ptrs, hipStream_t s) {
    const int dev = current_device();
    // the fetch ring (or a chunk's sums where they change hands through LDS), and never less than what
    // keeps a second workgroup off the CU
    const int lds = std::max(kPhasedLdsBytes, lds_vectors * threads * 16);
    if (!allowed[dev].load(std::memory_order_relaxed)) {
        hipError_t rc = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, lds);
        if (rc != hipSuccess) return (int)rc;
        allowed[dev].store(1, std::memory_order_relaxed);
    }
    int64_t grid = L.num_blocks > 0 ? L.num_blocks : current_cus();
    if (grid > L.total_chunks) grid = L.total_chunks;
    if (grid <= 0) return 0;
    hipLaunchKernelGGL(kernel, dim3((unsigned)grid), dim3(threads), (size_t)lds, s, L, ptrs);
    return (int)hipGetLastError();
}

template <int DT>
static int launch_phased_dt(const PhasedLaunch& L, const RankPtrs& ptrs, hipStream_t s) {
    static std::atomic<int> allowed[8][kMaxDevices];
    // integer sums never arrive as trees (the planner re-associates them into chains), and the 8-bit
    // floats' arithmetic leaves no registers for the tree code
    constexpr bool kNoTrees = DT == PCCL_I32 || DT == PCCL_F8E4M3 || DT == PCCL_F8E5M2;
    switch (L.shape) {
        case 0: return launch_phased_kernel(phased_kernel<DT, 512, 16, 4, 0, 2, false>, allowed[0], 512, 4, L, ptrs, s);
        case 1: return launch_phased_kernel(phased_kernel<DT, 256, 32, 8, 1, 2, false>, allowed[1], 256, 8, L, ptrs, s);
        case 2:
            if constexpr (kNoTrees) return (int)hipErrorInvalidValue;
            else return launch_phased_kernel(phased_kernel<DT, 256, 32, 8, 1, 2, true>, allowed[2], 256, 8, L, ptrs, s);
        case 3: return launch_phased_kernel(phased_kernel<DT, 256, 32, 8, 2, 2, false>, allowed[3], 256, 32, L, ptrs, s);
        case 4: return launch_phased_kernel(phased_kernel_pairs<DT, 512, 16, 4, 2, 2>, allowed[4], 512, 4, L, ptrs, s);   // two sweeps per write phase
        case 5: {
            // the grid has to be what the host chose the group for
            int64_t grid = L.num_blocks > 0 ? L.num_blocks : current_cus();
            if (grid > L.total_chunks) grid = L.total_chunks;
            if (L.group < 1 || (L.group & (L.group - 1)) || grid % L.group || L.total_chunks % L.group) return (int)hipErrorInvalidValue;
            if (L.group_segs > 1) {
                if (L.seg_chunks <= 0 || L.seg_chunks * L.group_segs != L.group) return (int)hipErrorInvalidValue;
                switch (L.group_segs) {
                    case 2: return launch_phased_kernel(phased_kernel_linear_rows<DT, 256, 32, 8, 2, 2>, allowed[6], 256, 8, L, ptrs, s);
                    case 4: return launch_phased_kernel(phased_kernel_linear_rows<DT, 256, 32, 8, 2, 4>, allowed[7], 256, 8, L, ptrs, s);
                    default: return (int)hipErrorInvalidValue;
                }
            }
            return launch_phased_kernel(phased_kernel_linear<DT, 256, 32, 8, 2>, allowed[5], 256, 8, L, ptrs, s);
        }
        default: return (int)hipErrorInvalidValue;
    }
}

int launch_phased(const PhasedLaunch& L, const RankPtrs& ptrs, void* stream) {
    hipStream_t s = (hipStream_t)stream;
    switch (L.dtype) {
        case PCCL_F32: return launch_phased_dt<PCCL_F32>(L, ptrs, s);
        case PCCL_F16: return launch_phased_dt<PCCL_F16>(L, ptrs, s);
        case PCCL_BF16: return launch_phased_dt<PCCL_BF16>(L, ptrs, s);
        case PCCL_I32: return launch_phased_dt<PCCL_I32>(L, ptrs, s);
        case PCCL_F8E4M3: return launch_phased_dt<PCCL_F8E4M3>(L, ptrs, s);
        case PCCL_F8E5M2: return launch_phased_dt<PCCL_F8E5M2>(L, ptrs, s);
        default: return (int)hipErrorInvalidValue;
    }
}

template <int DT>
static int launch_persistent_dt(const StepwiseLaunch& L, const RankPtrs& ptrs, hipStream_t s) {
    // Every workgroup must be resident at once.  A workgroup is one wave per SIMD; a SIMD holds 512
    // vector registers per lane and 800 scalar registers.  The kernel is compiled for 8 waves per
    // SIMD (amdgpu_waves_per_eu: at most 64 vector and 96 scalar registers); take the smallest of
    // that, the bound from the vector registers it reports and what the runtime says.  (A form of
    // this kernel that needed 100 scalar registers fitted only 7 times per CU while the runtime's
    // estimate said 8: the grid was one workgroup per CU too large and waits expired.)
    static std::atomic<int> cached_per_cu[kMaxDevices];   // per instantiation and device; the queries are made once
    const int dev = current_device();
    int per_cu = cached_per_cu[dev].load(std::memory_order_relaxed);
    if (per_cu == 0) {
        if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, persistent_kernel<DT>, kThreads, 0) != hipSuccess || per_cu <= 0) per_cu = 1;
        hipFuncAttributes attr;
        if (hipFuncGetAttributes(&attr, reinterpret_cast<const void*>(persistent_kernel<DT>)) == hipSuccess && attr.numRegs > 0) {
            const int by_vgpr = 512 / ((attr.numRegs + 7) / 8 * 8);
            if (by_vgpr < per_cu) per_cu = by_vgpr;
        }
        if (per_cu > 8) per_cu = 8;
        if (per_cu < 1) per_cu = 1;
        cached_per_cu[dev].store(per_cu, std::memory_order_relaxed);
    }
    const int resident = current_cus() * per_cu;
    // Default: 4 workgroups per CU.  On the headline graph 3, 4 and 5 per CU take 3.05 to 3.07 ms,
    // 8 per CU 3.10 ms, 2 per CU 3.34 ms (32 KiB items).
    const int wanted = L.num_blocks > 0 ? L.num_blocks : current_cus() * 4;
    int grid = wanted < resident ? wanted : resident;
    if (grid > L.num_items) grid = L.num_items;
    if (grid <= 0) return 0;
    hipLaunchKernelGGL((persistent_kernel<DT>), dim3(grid), dim3(kThreads), 0, s, L, ptrs);
    return (int)hipGetLastError();
}

int launch_persistent(const StepwiseLaunch& L, const RankPtrs& ptrs, void* stream) {
    hipStream_t s = (hipStream_t)stream;
    if (L.epoch == 0) {   // the launch number comes from the device-side counter: advance it first
        hipLaunchKernelGGL(advance_graph_epoch_kernel, dim3(1), dim3(kThreads), 0, s, L.state, L.num_items + L.num_ops + 1,
                           L.graph_epoch_limit > 0 ? L.graph_epoch_limit : kGraphEpochLimit);
        hipError_t rc = hipGetLastError();
        if (rc != hipSuccess) return (int)rc;
    }
    switch (L.dtype) {
        case PCCL_F32: return launch_persistent_dt<PCCL_F32>(L, ptrs, s);
        case PCCL_F16: return launch_persistent_dt<PCCL_F16>(L, ptrs, s);
        case PCCL_BF16: return launch_persistent_dt<PCCL_BF16>(L, ptrs, s);
        case PCCL_I32: return launch_persistent_dt<PCCL_I32>(L, ptrs, s);
        case PCCL_F8E4M3: return launch_persistent_dt<PCCL_F8E4M3>(L, ptrs, s);
        case PCCL_F8E5M2: return launch_persistent_dt<PCCL_F8E5M2>(L, ptrs, s);
        default: return (int)hipErrorInvalidValue;
    }
}

template <int DT>
static int launch_level_dt(const StepwiseLaunch& L, int item_begin, int item_end, const RankPtrs& ptrs, hipStream_t s) {
    int n = item_end - item_begin;
    if (n <= 0) return 0;
    constexpr int ES = ElemBytes<DT>::value;
    int subs = (int)((L.tile_elems * ES + kPrimTileBytes - 1) / kPrimTileBytes);
    int64_t total = (int64_t)n * subs;
    const int run = run_for_tiles(total);
    int64_t cap = L.num_blocks > 0 ? L.num_blocks : ((int64_t)1 << 30);
    const int64_t want = span_tiles(total, run);
    int grid = (int)(want < cap ? want : cap);
    hipLaunchKernelGGL((level_kernel<DT>), dim3(grid), dim3(kThreads), 0, s, L, item_begin, item_end, subs, run, ptrs);
    return (int)hipGetLastError();
}

int launch_level(const StepwiseLaunch& L, int item_begin, int item_end, const RankPtrs& ptrs, void* stream) {
    hipStream_t s = (hipStream_t)stream;
    switch (L.dtype) {
        case PCCL_F32: return launch_level_dt<PCCL_F32>(L, item_begin, item_end, ptrs, s);
        case PCCL_F16: return launch_level_dt<PCCL_F16>(L, item_begin, item_end, ptrs, s);
        case PCCL_BF16: return launch_level_dt<PCCL_BF16>(L, item_begin, item_end, ptrs, s);
        case PCCL_I32: return launch_level_dt<PCCL_I32>(L, item_begin, item_end, ptrs, s);
        case PCCL_F8E4M3: return launch_level_dt<PCCL_F8E4M3>(L, item_begin, item_end, ptrs, s);
        case PCCL_F8E5M2: return launch_level_dt<PCCL_F8E5M2>(L, item_begin, item_end, ptrs, s);
        default: return (int)hipErrorInvalidValue;
    }
}

int launch_reduce(int dtype, int redop, const void* a, const void* b, void* c, size_t n, void* stream) {
    if (n == 0) return 0;
    hipStream_t s = (hipStream_t)stream;
    const char* pa = (const char*)a; const char* pb = (const char*)b; char* pc = (char*)c;
    int es = (dtype == PCCL_F32 || dtype == PCCL_I32) ? 4 : (dtype == PCCL_F16 || dtype == PCCL_BF16) ? 2 : 1;
    const int64_t ntiles = ((int64_t)n * es + kPrimTileBytes - 1) / kPrimTileBytes + 1;   // + 1: tiles are anchored at aligned addresses
    const int run = run_for_tiles(ntiles);
    int grid = grid_for_tiles(ntiles, run);
    switch (dtype) {
        case PCCL_F32: hipLaunchKernelGGL((reduce_kernel<PCCL_F32>), dim3(grid), dim3(kThreads), 0, s, pa, pb, pc, (int64_t)n, redop, run); break;
        case PCCL_F16: hipLaunchKernelGGL((reduce_kernel<PCCL_F16>), dim3(grid), dim3(kThreads), 0, s, pa, pb, pc, (int64_t)n, redop, run); break;
        case PCCL_BF16: hipLaunchKernelGGL((reduce_kernel<PCCL_BF16>), dim3(grid), dim3(kThreads), 0, s, pa, pb, pc, (int64_t)n, redop, run); break;
        case PCCL_I32: hipLaunchKernelGGL((reduce_kernel<PCCL_I32>), dim3(grid), dim3(kThreads), 0, s, pa, pb, pc, (int64_t)n, redop, run); break;
        case PCCL_F8E4M3: hipLaunchKernelGGL((reduce_kernel<PCCL_F8E4M3>), dim3(grid), dim3(kThreads), 0, s, pa, pb, pc, (int64_t)n, redop, run); break;
        case PCCL_F8E5M2: hipLaunchKernelGGL((reduce_kernel<PCCL_F8E5M2>), dim3(grid), dim3(kThreads), 0, s, pa, pb, pc, (int64_t)n, redop, run); break;
        default: return (int)hipErrorInvalidValue;
    }
    return (int)hipGetLastError();
}

int launch_copy_bytes(const void* src, void* dst, size_t nbytes, void* stream) {
    if (nbytes == 0) return 0;
    const int64_t ntiles = ((int64_t)nbytes + kPrimTileBytes - 1) / kPrimTileBytes + 1;   // + 1: tiles are anchored at aligned addresses
    const int run = run_for_tiles(ntiles);
    hipLaunchKernelGGL(copy_kernel, dim3(grid_for_tiles(ntiles, run)), dim3(kThreads), 0, (hipStream_t)stream, (const char*)src, (char*)dst, (int64_t)nbytes, run);
    return (int)hipGetLastError();
}

int launch_stage(const RankPtrs& src, const RankPtrs& dst, const StageOffsets& off, int R, size_t bytes, void* stream) {
    if (bytes == 0 || R <= 0) return 0;
    int64_t ntiles = ((int64_t)bytes + kPrimTileBytes - 1) / kPrimTileBytes + 1;   // + 1: tiles are anchored at aligned addresses
    const int run = run_for_tiles(ntiles);
    const int64_t cap = 1 << 24, want = span_tiles(ntiles, run);
    int gx = (int)(want < cap ? want : cap);   // a multiple of 8, so that blockIdx.x % 8 is the XCD in every row
    hipLaunchKernelGGL(stage_kernel, dim3(gx, R), dim3(kThreads), 0, (hipStream_t)stream, src, dst, off, (int64_t)bytes, run);
    return (int)hipGetLastError();
}

int launch_gather(const DevGatherCopy* copies, int n, int64_t total_tiles, int copy_tiles, const RankPtrs& src, const RankPtrs& dst, void* stream) {
    if (n <= 0 || total_tiles <= 0) return 0;
    const int run = run_for_tiles(total_tiles);
    hipLaunchKernelGGL(gather_kernel, dim3(grid_for_tiles(total_tiles, run)), dim3(kThreads), 0, (hipStream_t)stream, copies, n, total_tiles, copy_tiles, src, dst, run);
    return (int)hipGetLastError();
}

// ------------------------------------------------------------------------------- static workspace
//
// Device memory of a stated, fixed size that exists from the moment the library is loaded: the
// persistent runner's tables and progress block of a call that may not allocate live here.  Every
// GPU the library runs on holds its own copy of the array at its own address; the array's name is
// a host-side stand-in, not a device address, so host code asks the runtime for the address once
// per device and from then on only ever uses that pointer.  Every call on a GPU shares that GPU's
// array, which keeps the last call's contents.
static __device__ __align__(256) unsigned char scratch[PCCL_HIP_STATIC_WORKSPACE_BYTES];

static std::atomic<void*> g_scratch_ptr[kMaxDevices];

int static_workspace(int device, void** ptr, size_t* bytes) {
    if (device < 0 || device >= kMaxDevices) return (int)hipErrorInvalidDevice;
    void* p = g_scratch_ptr[device].load(std::memory_order_acquire);
    if (!p) {
        int cur = -1;
        hipError_t rc = hipGetDevice(&cur);
        if (rc != hipSuccess) return (int)rc;
        if (cur != device) return (int)hipErrorInvalidDevice;   // the address is asked for with its device current
        rc = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (rc != hipSuccess) return (int)rc;
        if (!p) return (int)hipErrorInvalidSymbol;
        g_scratch_ptr[device].store(p, std::memory_order_release);
    }
    *ptr = p;
    *bytes = sizeof(scratch);
    return 0;
}

// Table bytes carried to the device by the kernel arguments themselves: no copy engine, no staging
// buffer, nothing allocated anywhere.
__global__ __launch_bounds__(kThreads) void table_write_kernel(TablePayload payload, uint64_t* dst, int nwords) {
    for (int i = threadIdx.x; i < nwords; i += kThreads) dst[i] = payload.w[i];
}

int launch_table_write(const void* src, size_t nbytes, void* dst, void* stream) {
    if (nbytes % 8 || (uintptr_t)dst % 8) return (int)hipErrorInvalidValue;
    const char* s = (const char*)src;
    char* d = (char*)dst;
    while (nbytes > 0) {
        TablePayload payload;
        const size_t n = nbytes < sizeof(payload.w) ? nbytes : sizeof(payload.w);
        std::memcpy(payload.w, s, n);
        hipLaunchKernelGGL(table_write_kernel, dim3(1), dim3(kThreads), 0, (hipStream_t)stream, payload, (uint64_t*)d, (int)(n / 8));
        hipError_t rc = hipGetLastError();
        if (rc != hipSuccess) return (int)rc;
        s += n; d += n; nbytes -= n;
    }
    return 0;
}

// item -> op map of the stepwise plan, rebuilt on the device from the op table (op k owns items
// [first_item, first_item + ntiles)).
__global__ __launch_bounds__(kThreads) void item_op_fill_kernel(const DevStepOp* ops, int num_ops, int32_t* item_op) {
    for (int k = blockIdx.x; k < num_ops; k += gridDim.x) {
        const int first = ops[k].first_item, n = ops[k].ntiles;
        for (int t = threadIdx.x; t < n; t += kThreads) item_op[first + t] = k;
    }
}

int launch_item_op_fill(const DevStepOp* ops, int num_ops, int32_t* item_op, void* stream) {
    if (num_ops <= 0) return 0;
    hipLaunchKernelGGL(item_op_fill_kernel, dim3(num_ops < 1024 ? num_ops : 1024), dim3(kThreads), 0, (hipStream_t)stream, ops, num_ops, item_op);
    return (int)hipGetLastError();
}

int launch_fill_zero(void* dst, size_t nbytes, void* stream) {
    int64_t nwords = (int64_t)(nbytes / 4);
    if (nwords == 0) return 0;
    int grid = (int)((nwords + kThreads - 1) / kThreads);
    if (grid > 1024) grid = 1024;
    hipLaunchKernelGGL(fill_zero_kernel, dim3(grid), dim3(kThreads), 0, (hipStream_t)stream, (uint32_t*)dst, nwords);
    return (int)hipGetLastError();
}

}  // namespace pccl_hip
