/*
 * pccl_oracle.c — CPU restatement of the reference's SM-executor data path.  TEST INFRASTRUCTURE ONLY.
 *
 * This file is the checker that the HIP executor is compared against.  It is never linked into,
 * imported by or called from the product library; only tests, the smoke check and the CPU-baseline
 * leg of the benchmark may use it.
 *
 * The reference has no CPU executor (csrc/plugins/host/host_device.cc:172-180 is an empty body), so
 * this is a restatement of what its CUDA kernels compute, one function per reference function:
 *
 *   oracle_add_*        Vec<T>::operator+ as used by vector_add_impl
 *                       (csrc/plugins/cuda/kernel/compute.h:46-72, vec.h:104-111 f32,
 *                        :170-177 f16 __hadd2, :232-239 bf16 __hadd2)
 *   run_reduce          executeReduce  (csrc/plugins/cuda/cuda_executor.cu:60-81)
 *                       c = self+off2, a = peers[peer]+off0, b = self+off1, element offsets
 *   run_copy            executeCopy    (csrc/plugins/cuda/cuda_executor.cu:83-101)
 *   notify / wait       executeNotify / executeWaitNotify (cuda_executor.cu:414-445):
 *                       notify = signals[target][id] += 1, wait = block while == 0, then -= 1
 *   pccl_oracle_run     the dependency-counter runner (cuda_executor.cu:498-510,526-918): an op
 *                       becomes ready when all its dependencies completed; each channel of each
 *                       rank runs one op at a time from a FIFO ready queue; a wait at the head of
 *                       a queue blocks that channel until its semaphore is positive.
 *
 * Parity status of each function (what pins it, beyond this file):
 *   f32 add            IEEE binary32 addition, round-to-nearest-even: C `float +`.  PINNED by numpy
 *                      float32 and torch CPU add in the tests.
 *   bf16 / f16 add     one correctly rounded add in the storage type.  Computed as
 *                      RNE(float(a)+float(b)); the float sum of two p-bit values rounds innocuously
 *                      because 24 >= 2p+2 (p = 8, 11).  PINNED by torch CPU bf16/f16 add over every
 *                      pair in a dense sample and by numpy float16.
 *   NaN results        canonical NaN (0x7FFFFFFF / 0x7FFF), the value PTX add.f32 / add.f16x2 /
 *                      add.bf16x2 produce.  PARITY UNPINNED (no CUDA device to confirm; taken from
 *                      the PTX ISA description of NaN payloads).
 *   fp8 add            e4m3 / e5m2 widened to f16, one f16 add, narrowed round-to-nearest-even with
 *                      saturation to the largest finite value (vec.h:272-426).  PINNED over all
 *                      65,536 operand pairs of both formats by torch CPU: float8 -> float16 views,
 *                      float16 add, clamp to +-max, float16 -> float8.  NaN results are written as
 *                      0x7F: PARITY UNPINNED.
 *   copy               memcpy.  PINNED trivially.
 *   signals + runner   counting semaphores.  PINNED by the closed forms of the reference's own
 *                      correctness script (tests/test_correctness.py:142-289) and by brute-force
 *                      evaluation of each schedule's per-element reduction order.
 *   counts carried     pccl_oracle_run_carry: the semaphore region outlives an execution and is
 *   over               shared by all operations of an engine (engine_c.cc:131-146, cleared only by
 *                      resetSignals :576-593).  The reference has no test of it; PINNED by known
 *                      answers that follow from executeWaitNotify / executeNotify alone: a wait with
 *                      no notify anywhere deadlocks from zero and passes, once per count, on what an
 *                      earlier execution left; the state after k executions of an operation with
 *                      n notifies and w waits on a semaphore is k (n - w); resetSignals restores
 *                      the deadlock (tests/test_oracle.py).
 *   tails              the reference drops the last n % (16/sizeof T) elements of every chunk and
 *                      issues unconditional 16-byte loads (compute.h:26,52; vec.h:25-28), so sizes
 *                      and offsets that are not multiples of 16 bytes have no defined reference
 *                      result.  This oracle processes all n elements at any alignment.  EXTENSION,
 *                      parity unpinned by the reference; pinned by closed forms.
 *   MAX / MIN, int32   the reference runtime ignores reduce_op and rejects int32.  EXTENSION: MAX and
 *                      MIN are IEEE 754-2019 maximum / minimum (NaN propagates, -0 < +0), pinned by
 *                      torch maximum / minimum / amax / amin and by known answers for the zeros.
 *
 * Build: gcc -O2 -fopenmp -shared -fPIC (see oracle/build.py).  No dependency on ROCm or torch.
 */
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#include <stdio.h>
#include <math.h>
#ifdef _OPENMP
#include <omp.h>
#endif

enum { DT_F32 = 0, DT_F16 = 1, DT_BF16 = 2, DT_F8E4M3 = 3, DT_F8E5M2 = 4, DT_I32 = 5 };
enum { RED_SUM = 0, RED_MAX = 1, RED_MIN = 2 };
enum { K_NOOP = 0, K_REDUCE = 1, K_COPY = 2, K_NOTIFY = 3, K_WAIT = 4 };

#define ORACLE_MAX_NEXT 8
#define ORACLE_NUM_SIGNALS 4096 /* include/common/config.h:24 — 4096 ints per rank */
#define ORACLE_MAX_CHANNELS 8   /* include/common/config.h:27 */

typedef struct {
    int32_t kind;
    int32_t index;
    int32_t channel;
    int32_t peer;    /* data: source rank; notify: target rank; wait: source rank (ignored) */
    int32_t off0;    /* reduce: remote_offset; copy: src_offset; signals: signal_id */
    int32_t off1;    /* reduce: src_offset;    copy: dst_offset */
    int32_t off2;    /* reduce: dst_offset */
    int32_t size;    /* elements */
    int32_t redop;
    int32_t ndeps;
    int32_t nnext;
    int32_t next[ORACLE_MAX_NEXT];
} oracle_op;

typedef struct {
    int64_t ops_executed;
    int64_t data_ops;
    int64_t bytes;        /* algorithmic bytes: reduce 3*n*esize, copy 2*n*esize */
    int32_t deadlocked;   /* 1 if the run stopped with blocked waits */
    int32_t residual;     /* number of (rank, id) semaphores left non-zero */
} oracle_stats;

static char g_err[512];
const char* pccl_oracle_last_error(void) { return g_err; }

int pccl_oracle_elem_size(int dtype) {
    switch (dtype) {
        case DT_F32: case DT_I32: return 4;
        case DT_F16: case DT_BF16: return 2;
        case DT_F8E4M3: case DT_F8E5M2: return 1;
        default: return 0;
    }
}

/* ---------------------------------------------------------------- scalar arithmetic */

static inline uint32_t f2u(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }
static inline float u2f(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }

static inline float oracle_add_f32(float a, float b) {
    float s = a + b;
    if (s != s) return u2f(0x7FFFFFFFu);
    return s;
}

static inline float bf16_to_f32(uint16_t h) { return u2f((uint32_t)h << 16); }

static inline uint16_t f32_to_bf16_rne(float f) {
    uint32_t u = f2u(f);
    if (f != f) return 0x7FFF;
    u += 0x7FFFu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}

static inline uint16_t oracle_add_bf16(uint16_t a, uint16_t b) {
    return f32_to_bf16_rne(bf16_to_f32(a) + bf16_to_f32(b));
}

static inline float f16_to_f32(uint16_t h) {
    uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1Fu;
    uint32_t man = h & 0x3FFu;
    if (exp == 0) {
        if (man == 0) return u2f(sign);
        /* subnormal: value = man * 2^-24 */
        float v = (float)man * (1.0f / 16777216.0f);
        return sign ? -v : v;
    }
    if (exp == 31) return u2f(sign | 0x7F800000u | (man << 13));
    return u2f(sign | ((exp + 112u) << 23) | (man << 13));
}

static inline uint16_t f32_to_f16_rne(float f) {
    uint32_t u = f2u(f);
    uint16_t sign = (uint16_t)((u >> 16) & 0x8000u);
    uint32_t abs = u & 0x7FFFFFFFu;
    if (abs > 0x7F800000u) return 0x7FFF;                 /* NaN -> canonical */
    if (abs >= 0x477FF000u) return (uint16_t)(sign | 0x7C00u); /* >= 65520 rounds to inf (also inf) */
    if (abs < 0x33000001u) return sign;                    /* <= 2^-25 rounds to zero (ties to even) */
    int32_t e = (int32_t)(abs >> 23) - 127;
    uint32_t m = (abs & 0x7FFFFFu) | 0x800000u;            /* 24-bit significand */
    int shift = (e < -14) ? (13 + (-14 - e)) : 13;         /* bits dropped */
    uint32_t kept = m >> shift;
    uint32_t rem = m & ((1u << shift) - 1u);
    uint32_t half = 1u << (shift - 1);
    if (rem > half || (rem == half && (kept & 1u))) kept++;
    uint32_t out;
    if (e < -14) out = kept;                               /* subnormal (may carry into normal) */
    else out = ((uint32_t)(e + 15) << 10) + (kept - 0x400u); /* carry propagates into exponent */
    return (uint16_t)(sign | out);
}

static inline uint16_t oracle_add_f16(uint16_t a, uint16_t b) {
    return f32_to_f16_rne(f16_to_f32(a) + f16_to_f32(b));
}

/* MAX / MIN (extension): IEEE 754-2019 maximum / minimum.  A NaN operand gives NaN (canonical);
 * -0 orders below +0, so the result does not depend on the order of the operands.  Operands that
 * compare equal are either bit-identical or the two zeros: AND of the bit patterns keeps +0 for the
 * maximum, OR keeps -0 for the minimum, and both leave identical patterns alone. */
static inline float sel_max_f32(float a, float b) {
    if (a != a || b != b) return u2f(0x7FFFFFFFu);
    if (a == b) return u2f(f2u(a) & f2u(b));
    return a > b ? a : b;
}
static inline float sel_min_f32(float a, float b) {
    if (a != a || b != b) return u2f(0x7FFFFFFFu);
    if (a == b) return u2f(f2u(a) | f2u(b));
    return a < b ? a : b;
}

/* fp8 (reference vec.h:272-426): both operands are widened to f16 (exact), added with one f16
 * rounding (__hadd2), and narrowed with __nv_cvt_halfraw2_to_fp8x2(..., __NV_SATFINITE, type):
 * round to nearest even, everything beyond the largest finite value - infinities included -
 * becomes that value with the sign kept.  E4M3 is the OCP "FN" format (bias 7, no infinities,
 * S.1111.111 is NaN, largest finite 448); E5M2 is IEEE-like (bias 15, largest finite 57344).
 * A NaN result is written as 0x7F in both formats: canonical choice, parity unpinned (no CUDA
 * device to confirm the payload the conversion instruction produces). */
static inline float fp8_to_f32(uint8_t v, int e5m2) {
    const int mbits = e5m2 ? 2 : 3, bias = e5m2 ? 15 : 7;
    const uint32_t sign = (uint32_t)(v & 0x80u) << 24;
    const int exp = (v & 0x7F) >> mbits, man = v & ((1 << mbits) - 1);
    if (e5m2) {
        if (exp == 31) return u2f(sign | (man ? 0x7FC00000u : 0x7F800000u));
    } else if ((v & 0x7F) == 0x7F) return u2f(sign | 0x7FC00000u);
    float mag;
    if (exp == 0) mag = ldexpf((float)man, 1 - bias - mbits);
    else mag = ldexpf((float)(man | (1 << mbits)), exp - bias - mbits);
    return sign ? -mag : mag;
}

static inline uint8_t f32_to_fp8_satfinite(float f, int e5m2) {
    const int mbits = e5m2 ? 2 : 3, bias = e5m2 ? 15 : 7;
    const uint8_t maxnorm = e5m2 ? 0x7B : 0x7E;
    if (f != f) return 0x7F;
    const uint8_t sign = (f2u(f) >> 31) ? 0x80 : 0x00;
    const double a = fabs((double)f);
    const double maxval = e5m2 ? 57344.0 : 448.0;
    if (a >= maxval) return sign | maxnorm;                 /* saturate (also +-inf) */
    if (a == 0.0) return sign;
    int e;
    (void)frexp(a, &e);                                     /* a = m * 2^e, m in [0.5, 1) */
    int ue = e - 1;                                         /* a in [2^ue, 2^(ue+1)) */
    if (ue < 1 - bias) ue = 1 - bias;                       /* subnormal range: fixed quantum */
    const double quantum = ldexp(1.0, ue - mbits);
    const double q = a / quantum;                           /* exact: power-of-two scaling */
    double fl = floor(q);
    const double rem = q - fl;
    if (rem > 0.5 || (rem == 0.5 && fmod(fl, 2.0) == 1.0)) fl += 1.0;
    /* fl is the significand in units of the quantum: in [0, 2^(mbits+1)] */
    int k = (int)fl;
    int be = ue + bias;                                     /* biased exponent if normal */
    if (ue == 1 - bias && k < (1 << mbits)) return sign | (uint8_t)k;          /* subnormal or zero */
    if (k == (2 << mbits)) { k >>= 1; be += 1; }            /* rounding carried into the exponent */
    uint8_t out = (uint8_t)((be << mbits) | (k - (1 << mbits)));
    if (out > maxnorm) out = maxnorm;                       /* cannot happen below maxval; guard */
    return sign | out;
}

static inline uint8_t oracle_red_fp8(uint8_t a, uint8_t b, int redop, int e5m2) {
    const float x = fp8_to_f32(a, e5m2), y = fp8_to_f32(b, e5m2);
    float r;
    if (redop == RED_SUM) r = f16_to_f32(f32_to_f16_rne(x + y));   /* = __hadd2 on the widened pair */
    else if (redop == RED_MAX) r = sel_max_f32(x, y);
    else r = sel_min_f32(x, y);
    return f32_to_fp8_satfinite(r, e5m2);
}

/* ---------------------------------------------------------------- vector ops over a range */

#define LOOP_HDR _Pragma("omp parallel for schedule(static) if (n > 65536)")

static void reduce_range(int dtype, int redop, const void* a, const void* b, void* c, int64_t n) {
    if (dtype == DT_F32) {
        const float* pa = a; const float* pb = b; float* pc = c;
        if (redop == RED_SUM) { LOOP_HDR for (int64_t i = 0; i < n; i++) pc[i] = oracle_add_f32(pa[i], pb[i]); }
        else if (redop == RED_MAX) { LOOP_HDR for (int64_t i = 0; i < n; i++) pc[i] = sel_max_f32(pa[i], pb[i]); }
        else { LOOP_HDR for (int64_t i = 0; i < n; i++) pc[i] = sel_min_f32(pa[i], pb[i]); }
    } else if (dtype == DT_I32) {
        const int32_t* pa = a; const int32_t* pb = b; int32_t* pc = c;
        if (redop == RED_SUM) { LOOP_HDR for (int64_t i = 0; i < n; i++) pc[i] = (int32_t)((uint32_t)pa[i] + (uint32_t)pb[i]); }
        else if (redop == RED_MAX) { LOOP_HDR for (int64_t i = 0; i < n; i++) pc[i] = pa[i] > pb[i] ? pa[i] : pb[i]; }
        else { LOOP_HDR for (int64_t i = 0; i < n; i++) pc[i] = pa[i] < pb[i] ? pa[i] : pb[i]; }
    } else if (dtype == DT_BF16) {
        const uint16_t* pa = a; const uint16_t* pb = b; uint16_t* pc = c;
        if (redop == RED_SUM) { LOOP_HDR for (int64_t i = 0; i < n; i++) pc[i] = oracle_add_bf16(pa[i], pb[i]); }
        else if (redop == RED_MAX) { LOOP_HDR for (int64_t i = 0; i < n; i++) pc[i] = f32_to_bf16_rne(sel_max_f32(bf16_to_f32(pa[i]), bf16_to_f32(pb[i]))); }
        else { LOOP_HDR for (int64_t i = 0; i < n; i++) pc[i] = f32_to_bf16_rne(sel_min_f32(bf16_to_f32(pa[i]), bf16_to_f32(pb[i]))); }
    } else if (dtype == DT_F16) {
        const uint16_t* pa = a; const uint16_t* pb = b; uint16_t* pc = c;
        if (redop == RED_SUM) { LOOP_HDR for (int64_t i = 0; i < n; i++) pc[i] = oracle_add_f16(pa[i], pb[i]); }
        else if (redop == RED_MAX) { LOOP_HDR for (int64_t i = 0; i < n; i++) pc[i] = f32_to_f16_rne(sel_max_f32(f16_to_f32(pa[i]), f16_to_f32(pb[i]))); }
        else { LOOP_HDR for (int64_t i = 0; i < n; i++) pc[i] = f32_to_f16_rne(sel_min_f32(f16_to_f32(pa[i]), f16_to_f32(pb[i]))); }
    } else if (dtype == DT_F8E4M3 || dtype == DT_F8E5M2) {
        const uint8_t* pa = a; const uint8_t* pb = b; uint8_t* pc = c;
        const int e5m2 = dtype == DT_F8E5M2;
        LOOP_HDR for (int64_t i = 0; i < n; i++) pc[i] = oracle_red_fp8(pa[i], pb[i], redop, e5m2);
    }
}

/* Exposed for unit tests of the arithmetic alone. */
int pccl_oracle_reduce(int dtype, int redop, const void* a, const void* b, void* c, int64_t n) {
    if (pccl_oracle_elem_size(dtype) == 0) {
        snprintf(g_err, sizeof g_err, "reduce: dtype %d not supported by the oracle", dtype);
        return -1;
    }
    reduce_range(dtype, redop, a, b, c, n);
    return 0;
}

int pccl_oracle_copy(int dtype, const void* src, void* dst, int64_t n) {
    int es = pccl_oracle_elem_size(dtype);
    if (!es) { snprintf(g_err, sizeof g_err, "copy: bad dtype %d", dtype); return -1; }
    memmove(dst, src, (size_t)n * es);
    return 0;
}

/* ---------------------------------------------------------------- the runner */

typedef struct { int* q; int head, tail, cap; } fifo;

static uint32_t lcg(uint32_t* s) { *s = *s * 1664525u + 1013904223u; return *s >> 8; }

/*
 * Run R per-rank graphs to completion.
 *   ops[r], nops[r]  rank r's operations; `index` values are positions in ops[r]
 *   bufs[r]          rank r's buffer of buf_elems elements (offsets index into it)
 *   sched_seed       0: drain each (rank, channel) queue in rank-major order;
 *                    otherwise visit (rank, channel) pairs in a seeded pseudo-random order,
 *                    one op per visit — results must not depend on it for a race-free graph
 *   threads          OpenMP threads for the element loops (<=0: library default)
 * Returns 0 on success, -1 bad argument / out-of-range access, -2 deadlock.
 */
int pccl_oracle_run_carry(int R, const int32_t* nops, const oracle_op* const* ops, int dtype,
                          void* const* bufs, int64_t buf_elems, uint32_t sched_seed, int threads,
                          int32_t* signals_io, oracle_stats* stats);

int pccl_oracle_run(int R, const int32_t* nops, const oracle_op* const* ops, int dtype,
                    void* const* bufs, int64_t buf_elems, uint32_t sched_seed, int threads,
                    oracle_stats* stats) {
    return pccl_oracle_run_carry(R, nops, ops, dtype, bufs, buf_elems, sched_seed, threads, NULL, stats);
}

/*
 * The same with the semaphores handed in and out: signals_io holds R x ORACLE_NUM_SIGNALS counts
 * (rank-major), read as the state the execution starts from and left as the state it ends in.  The
 * reference keeps one signal region per engine for all registered operations and clears it only in
 * Engine::resetSignals (csrc/engine_c.cc:576-593): counts that one execution leaves above zero are
 * what the waits of the next execution, of any operation, find (cuda_executor.cu:425-445: a wait
 * passes on a positive count and takes one).  NULL: start from zero and forget, as pccl_oracle_run.
 */
int pccl_oracle_run_carry(int R, const int32_t* nops, const oracle_op* const* ops, int dtype,
                          void* const* bufs, int64_t buf_elems, uint32_t sched_seed, int threads,
                          int32_t* signals_io, oracle_stats* stats) {
    int es = pccl_oracle_elem_size(dtype);
    if (R <= 0 || !es) { snprintf(g_err, sizeof g_err, "bad R=%d or dtype=%d", R, dtype); return -1; }
#ifdef _OPENMP
    if (threads > 0) omp_set_num_threads(threads);
#endif
    oracle_stats st; memset(&st, 0, sizeof st);
    int rc = 0;
    int32_t* signals = signals_io ? signals_io : calloc((size_t)R * ORACLE_NUM_SIGNALS, sizeof(int32_t));
    int** remaining = calloc(R, sizeof(int*));
    fifo* queues = calloc((size_t)R * ORACLE_MAX_CHANNELS, sizeof(fifo));
    int64_t total = 0, done = 0;

    for (int r = 0; r < R; r++) {
        remaining[r] = malloc(sizeof(int) * (nops[r] > 0 ? nops[r] : 1));
        for (int c = 0; c < ORACLE_MAX_CHANNELS; c++) {
            fifo* f = &queues[r * ORACLE_MAX_CHANNELS + c];
            f->cap = nops[r] + 1; f->q = malloc(sizeof(int) * f->cap); f->head = f->tail = 0;
        }
        for (int i = 0; i < nops[r]; i++) {
            const oracle_op* o = &ops[r][i];
            if (o->channel < 0 || o->channel >= ORACLE_MAX_CHANNELS || o->nnext > ORACLE_MAX_NEXT) {
                snprintf(g_err, sizeof g_err, "rank %d op %d: channel %d / nnext %d out of range", r, i, o->channel, o->nnext);
                rc = -1; goto out;
            }
            for (int k = 0; k < o->nnext; k++)
                if (o->next[k] < 0 || o->next[k] >= nops[r]) {
                    snprintf(g_err, sizeof g_err, "rank %d op %d: next_ops[%d]=%d out of range", r, i, k, o->next[k]);
                    rc = -1; goto out;
                }
            remaining[r][i] = o->ndeps;
            total++;
        }
        /* seed: zero-dependency ops in index order (cuda_executor.cu:581-590) */
        for (int i = 0; i < nops[r]; i++)
            if (ops[r][i].ndeps == 0) { fifo* f = &queues[r * ORACLE_MAX_CHANNELS + ops[r][i].channel]; f->q[f->tail++] = i; }
    }

    int nq = R * ORACLE_MAX_CHANNELS;
    int* order = malloc(sizeof(int) * nq);
    for (int i = 0; i < nq; i++) order[i] = i;
    uint32_t rng = sched_seed;

    while (done < total) {
        int progressed = 0;
        if (sched_seed) for (int i = nq - 1; i > 0; i--) { int j = lcg(&rng) % (i + 1); int t = order[i]; order[i] = order[j]; order[j] = t; }
        for (int qi = 0; qi < nq; qi++) {
            int r = order[qi] / ORACLE_MAX_CHANNELS;
            fifo* f = &queues[order[qi]];
            while (f->head < f->tail) {
                int i = f->q[f->head];
                const oracle_op* o = &ops[r][i];
                if (o->kind == K_WAIT) {
                    if (o->off0 < 0 || o->off0 >= ORACLE_NUM_SIGNALS) { snprintf(g_err, sizeof g_err, "rank %d op %d: signal id %d", r, i, o->off0); rc = -1; goto out2; }
                    int32_t* s = &signals[(size_t)r * ORACLE_NUM_SIGNALS + o->off0];
                    if (*s <= 0) break;           /* blocked: the channel stalls on this wait */
                    *s -= 1;
                } else if (o->kind == K_NOTIFY) {
                    if (o->peer < 0 || o->peer >= R || o->off0 < 0 || o->off0 >= ORACLE_NUM_SIGNALS) { snprintf(g_err, sizeof g_err, "rank %d op %d: notify target %d id %d", r, i, o->peer, o->off0); rc = -1; goto out2; }
                    signals[(size_t)o->peer * ORACLE_NUM_SIGNALS + o->off0] += 1;
                } else if (o->kind == K_REDUCE || o->kind == K_COPY) {
                    int64_t n = o->size;
                    int bad = o->peer < 0 || o->peer >= R || n < 0 || o->off0 < 0 || o->off1 < 0 ||
                              (int64_t)o->off0 + n > buf_elems || (int64_t)o->off1 + n > buf_elems;
                    if (o->kind == K_REDUCE) bad = bad || o->off2 < 0 || (int64_t)o->off2 + n > buf_elems;
                    if (bad) { snprintf(g_err, sizeof g_err, "rank %d op %d: range outside the %lld-element buffer", r, i, (long long)buf_elems); rc = -1; goto out2; }
                    char* self = bufs[r]; const char* peer = bufs[o->peer];
                    if (o->kind == K_REDUCE) {
                        reduce_range(dtype, o->redop, peer + (int64_t)o->off0 * es, self + (int64_t)o->off1 * es,
                                     self + (int64_t)o->off2 * es, n);
                        st.bytes += 3 * n * es;
                    } else {
                        memmove(self + (int64_t)o->off1 * es, peer + (int64_t)o->off0 * es, (size_t)n * es);
                        st.bytes += 2 * n * es;
                    }
                    st.data_ops++;
                }
                f->head++;
                done++; st.ops_executed++; progressed = 1;
                for (int k = 0; k < o->nnext; k++) {
                    int nx = o->next[k];
                    if (--remaining[r][nx] == 0) { fifo* g = &queues[r * ORACLE_MAX_CHANNELS + ops[r][nx].channel]; g->q[g->tail++] = nx; }
                }
                if (sched_seed) break;             /* one op per visit in randomized mode */
            }
        }
        if (!progressed) {
            st.deadlocked = 1;
            snprintf(g_err, sizeof g_err, "deadlock: %lld of %lld ops executed, remaining channels blocked on waits or unmet dependencies",
                     (long long)done, (long long)total);
            rc = -2;
            break;
        }
    }
    for (size_t i = 0; i < (size_t)R * ORACLE_NUM_SIGNALS; i++) if (signals[i]) st.residual++;
out2:
    free(order);
out:
    for (int r = 0; r < R; r++) {
        if (remaining[r]) free(remaining[r]);
        for (int c = 0; c < ORACLE_MAX_CHANNELS; c++) free(queues[r * ORACLE_MAX_CHANNELS + c].q);
    }
    free(remaining); free(queues);
    if (!signals_io) free(signals);
    if (stats) *stats = st;
    return rc;
}

int pccl_oracle_sizeof_op(void) { return (int)sizeof(oracle_op); }
