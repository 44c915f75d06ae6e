/*
 * jl_cpu_path.c -- TEST / MEASUREMENT INFRASTRUCTURE ONLY.
 *
 * A restatement, with compiler intrinsics, of the reference's host path for the
 * packed decode matvec, so bench.py can time "what jitllm's own CPU tier does"
 * on the GPU box's host cores next to the GPU kernel.  The reference emits this
 * code at run time from Go (there is no Go toolchain here), so this is a port,
 * not the reference's binary:
 *
 *   activation quantizer   jit/cpu/quantdrive.go:78-161 (spec internal/oracle/quantize.go:80-119)
 *   fused packed matvec    jit/cpu/packedfused.go:54-367: sub-block major over the
 *                          [sub-block][word][row] planes, eight rows per 256-bit
 *                          register, one VPDPBUSD per (word, nibble field) into an
 *                          int32 accumulator, then out = fma(float(iacc), d*sc*d_a, out)
 *                          and the format's bias term; out accumulated in memory
 *   dot instruction        256-bit AVX-VNNI VPDPBUSD, or VPMADDUBSW+VPMADDWD where the
 *                          host lacks it (jit/cpu/prevnni.go:32-56); no AVX-512 tier
 *   row chunking           engine/nn/packed.go:82-119, 415-420: balanced row shares,
 *                          rounded to 16 outputs, one share per worker
 *   worker pool            engine/sched/pool.go:158: spinning workers, one region at a time
 *
 * Formats: Q4_K, Q8_0, Q6_K (the decode configurations).  Nothing in the product
 * library links or calls this file.
 */
#define _GNU_SOURCE
#include <immintrin.h>
#include <pthread.h>
#include <sched.h>
#include <stdatomic.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#include <time.h>

enum { T_Q8_0 = 8, T_Q4_K = 12, T_Q6_K = 14 };

typedef struct {
    int type;
    const uint32_t *qs, *d, *sc;
    const int8_t *a;      /* int8 activations [k] */
    const float *as;      /* [k/32] */
    const float *sum32;   /* [k/32]  sum of q per 32 */
    const float *sum16;   /* [k/16] */
    float *out;
    int nrows, k;
} job_t;

typedef struct pool {
    int nthreads;
    pthread_t *th;
    _Atomic int gen, done, quit;
    job_t job;
    int has_vnni;
    /* quantized activation scratch */
    int8_t *a;
    float *as, *sum32, *sum16;
    int cap_k;
} pool_t;

typedef struct { pool_t *p; int id; } warg_t;

/* ------------------------------------------------------------------ dots */

__attribute__((target("avx2,avxvnni"))) static inline __m256i dp_vnni(__m256i acc, __m256i u, __m256i s) {
    return _mm256_dpbusd_avx_epi32(acc, u, s);
}
__attribute__((target("avx2"))) static inline __m256i dp_vex(__m256i acc, __m256i u, __m256i s) {
    __m256i p = _mm256_maddubs_epi16(u, s);
    return _mm256_add_epi32(acc, _mm256_madd_epi16(p, _mm256_set1_epi16(1)));
}

/* Q4_K/Q5_K stream field (sub s, min) of eight rows: jit/gpu/kernels/scstream.go:32-52 */
#define SC_FIELD(ws, s, min, out)                                                        \
    do {                                                                                 \
        int f_ = 2 * (s) + (min), w_ = f_ * 6 / 32, b_ = f_ * 6 % 32;                     \
        if (b_ <= 26)                                                                    \
            out = _mm256_and_si256(_mm256_srli_epi32(ws[w_], b_), _mm256_set1_epi32(63)); \
        else                                                                             \
            out = _mm256_and_si256(                                                      \
                _mm256_or_si256(_mm256_srli_epi32(ws[w_], b_),                           \
                                _mm256_slli_epi32(ws[w_ + 1], 32 - b_)),                 \
                _mm256_set1_epi32(63));                                                  \
    } while (0)

#define ROWS_BODY(DP, TARGET)                                                                      \
    __attribute__((target(TARGET))) static void rows_q4k_##DP(const job_t *j, int lo, int hi) {    \
        const int nrows = j->nrows, nsub = j->k / 32;                                              \
        const __m256i m4 = _mm256_set1_epi32(0x0F0F0F0F);                                          \
        for (int r = lo; r < hi; r += 8) _mm256_storeu_ps(j->out + r, _mm256_setzero_ps());        \
        for (int si = 0; si < nsub; si++) {                                                        \
            const int sup = si >> 3, s = si & 7;                                                   \
            const uint32_t *a32 = (const uint32_t *)(j->a + si * 32);                              \
            const __m256 da = _mm256_set1_ps(j->as[si]);                                           \
            const __m256 bsum = _mm256_set1_ps(j->sum32[si] * j->as[si]);                          \
            __m256i al[4], ah[4];                                                                  \
            for (int w = 0; w < 4; w++) {                                                          \
                al[w] = _mm256_set1_epi32((int)a32[w]);                                            \
                ah[w] = _mm256_set1_epi32((int)a32[4 + w]);                                        \
            }                                                                                      \
            for (int r = lo; r < hi; r += 8) {                                                     \
                __m256i iacc = _mm256_setzero_si256();                                             \
                for (int w = 0; w < 4; w++) {                                                      \
                    __m256i pay = _mm256_loadu_si256(                                              \
                        (const __m256i *)(j->qs + ((size_t)si * 4 + w) * nrows + r));              \
                    iacc = dp_##DP(iacc, _mm256_and_si256(pay, m4), al[w]);                        \
                    iacc = dp_##DP(iacc, _mm256_and_si256(_mm256_srli_epi32(pay, 4), m4), ah[w]);  \
                }                                                                                  \
                __m256i dw = _mm256_loadu_si256((const __m256i *)(j->d + (size_t)sup * nrows + r)); \
                __m256i dlo = _mm256_and_si256(dw, _mm256_set1_epi32(0xFFFF));                     \
                __m256i dhi = _mm256_srli_epi32(dw, 16);                                           \
                __m256 d = _mm256_cvtph_ps(_mm256_castsi256_si128(_mm256_permute4x64_epi64(        \
                    _mm256_packus_epi32(dlo, dlo), 0xD8)));                                        \
                __m256 dmin = _mm256_cvtph_ps(_mm256_castsi256_si128(_mm256_permute4x64_epi64(     \
                    _mm256_packus_epi32(dhi, dhi), 0xD8)));                                        \
                __m256i ws[3], scv, mv;                                                            \
                for (int w = 0; w < 3; w++)                                                        \
                    ws[w] = _mm256_loadu_si256(                                                    \
                        (const __m256i *)(j->sc + ((size_t)sup * 3 + w) * nrows + r));             \
                SC_FIELD(ws, s, 0, scv);                                                           \
                SC_FIELD(ws, s, 1, mv);                                                            \
                __m256 sc = _mm256_mul_ps(_mm256_mul_ps(d, _mm256_cvtepi32_ps(scv)), da);          \
                __m256 o = _mm256_loadu_ps(j->out + r);                                            \
                o = _mm256_fmadd_ps(_mm256_cvtepi32_ps(iacc), sc, o);                              \
                o = _mm256_fnmadd_ps(_mm256_mul_ps(dmin, _mm256_cvtepi32_ps(mv)), bsum, o);        \
                _mm256_storeu_ps(j->out + r, o);                                                   \
            }                                                                                      \
        }                                                                                          \
    }                                                                                              \
    __attribute__((target(TARGET))) static void rows_q8_##DP(const job_t *j, int lo, int hi) {     \
        const int nrows = j->nrows, nsub = j->k / 32, dstride = (nrows + 1) / 2;                   \
        const __m256i flip = _mm256_set1_epi32((int)0x80808080u);                                  \
        for (int r = lo; r < hi; r += 8) _mm256_storeu_ps(j->out + r, _mm256_setzero_ps());        \
        for (int si = 0; si < nsub; si++) {                                                        \
            const uint32_t *a32 = (const uint32_t *)(j->a + si * 32);                              \
            const __m256 da = _mm256_set1_ps(j->as[si]);                                           \
            const __m256 corr = _mm256_set1_ps(-128.0f * j->sum32[si]);                            \
            __m256i av[8];                                                                         \
            for (int w = 0; w < 8; w++) av[w] = _mm256_set1_epi32((int)a32[w]);                    \
            for (int r = lo; r < hi; r += 8) {                                                     \
                __m256i iacc = _mm256_setzero_si256();                                             \
                for (int w = 0; w < 8; w++) {                                                      \
                    __m256i pay = _mm256_loadu_si256(                                              \
                        (const __m256i *)(j->qs + ((size_t)si * 8 + w) * nrows + r));              \
                    iacc = dp_##DP(iacc, _mm256_xor_si256(pay, flip), av[w]);                      \
                }                                                                                  \
                /* two rows share a d word: eight rows = four words = eight halves in row order */ \
                __m128i dh = _mm_loadu_si128((const __m128i *)(j->d + (size_t)si * dstride + r / 2)); \
                __m256 s = _mm256_mul_ps(_mm256_cvtph_ps(dh), da);                                 \
                __m256 o = _mm256_loadu_ps(j->out + r);                                            \
                o = _mm256_fmadd_ps(_mm256_add_ps(_mm256_cvtepi32_ps(iacc), corr), s, o);          \
                _mm256_storeu_ps(j->out + r, o);                                                   \
            }                                                                                      \
        }                                                                                          \
    }                                                                                              \
    __attribute__((target(TARGET))) static void rows_q6k_##DP(const job_t *j, int lo, int hi) {    \
        const int nrows = j->nrows, nsub = j->k / 16;                                              \
        const __m256i m4 = _mm256_set1_epi32(0x0F0F0F0F), m2 = _mm256_set1_epi32(0x03030303);      \
        for (int r = lo; r < hi; r += 8) _mm256_storeu_ps(j->out + r, _mm256_setzero_ps());        \
        for (int si = 0; si < nsub; si++) {                                                        \
            const int sup = si >> 4;                                                               \
            const uint32_t *a32 = (const uint32_t *)(j->a + si * 16);                              \
            const __m256 da = _mm256_set1_ps(j->as[si / 2]);                                       \
            const __m256 corr = _mm256_set1_ps(-32.0f * j->sum16[si]);                             \
            __m256i al[2], ah[2];                                                                  \
            for (int w = 0; w < 2; w++) {                                                          \
                al[w] = _mm256_set1_epi32((int)a32[w]);                                            \
                ah[w] = _mm256_set1_epi32((int)a32[2 + w]);                                        \
            }                                                                                      \
            for (int r = lo; r < hi; r += 8) {                                                     \
                const uint32_t *base = j->qs + (size_t)si * 3 * nrows + r;                         \
                __m256i hiw = _mm256_loadu_si256((const __m256i *)(base + 2 * (size_t)nrows));     \
                __m256i iacc = _mm256_setzero_si256();                                             \
                for (int w = 0; w < 2; w++) {                                                      \
                    __m256i pay = _mm256_loadu_si256((const __m256i *)(base + (size_t)w * nrows)); \
                    __m256i lo4 = _mm256_and_si256(pay, m4);                                       \
                    __m256i hi4 = _mm256_and_si256(_mm256_srli_epi32(pay, 4), m4);                 \
                    __m256i lo2 = _mm256_and_si256(_mm256_srli_epi32(hiw, 2 * w), m2);             \
                    __m256i hi2 = _mm256_and_si256(_mm256_srli_epi32(hiw, 4 + 2 * w), m2);         \
                    iacc = dp_##DP(iacc, _mm256_or_si256(lo4, _mm256_slli_epi32(lo2, 4)), al[w]);  \
                    iacc = dp_##DP(iacc, _mm256_or_si256(hi4, _mm256_slli_epi32(hi2, 4)), ah[w]);  \
                }                                                                                  \
                __m256i dw = _mm256_loadu_si256((const __m256i *)(j->d + (size_t)sup * nrows + r)); \
                __m256i dlo = _mm256_and_si256(dw, _mm256_set1_epi32(0xFFFF));                     \
                __m256 d = _mm256_cvtph_ps(_mm256_castsi256_si128(_mm256_permute4x64_epi64(        \
                    _mm256_packus_epi32(dlo, dlo), 0xD8)));                                        \
                __m256i sw = _mm256_loadu_si256(                                                   \
                    (const __m256i *)(j->sc + (size_t)(si / 4) * nrows + r));                      \
                __m256i scb = _mm256_sub_epi32(                                                    \
                    _mm256_and_si256(_mm256_srli_epi32(sw, 8 * (si % 4)), _mm256_set1_epi32(0xFF)), \
                    _mm256_set1_epi32(128));                                                       \
                __m256 s = _mm256_mul_ps(_mm256_mul_ps(d, _mm256_cvtepi32_ps(scb)), da);           \
                __m256 o = _mm256_loadu_ps(j->out + r);                                            \
                o = _mm256_fmadd_ps(_mm256_add_ps(_mm256_cvtepi32_ps(iacc), corr), s, o);          \
                _mm256_storeu_ps(j->out + r, o);                                                   \
            }                                                                                      \
        }                                                                                          \
    }

ROWS_BODY(vnni, "avx2,fma,f16c,avxvnni")
ROWS_BODY(vex, "avx2,fma,f16c")

static void run_rows(const pool_t *p, const job_t *j, int lo, int hi) {
    if (lo >= hi) return;
    switch (j->type) {
    case T_Q4_K: p->has_vnni ? rows_q4k_vnni(j, lo, hi) : rows_q4k_vex(j, lo, hi); break;
    case T_Q8_0: p->has_vnni ? rows_q8_vnni(j, lo, hi) : rows_q8_vex(j, lo, hi); break;
    case T_Q6_K: p->has_vnni ? rows_q6k_vnni(j, lo, hi) : rows_q6k_vex(j, lo, hi); break;
    }
}

/* Worker w's share of the rows: balanced, rounded to 16 outputs (one cache line),
 * engine/nn/packed.go:415-420. */
static void share(const job_t *j, int nthreads, int w, int *lo, int *hi) {
    int groups = (j->nrows + 15) / 16;
    int per = (groups + nthreads - 1) / nthreads;
    *lo = w * per * 16;
    *hi = (w + 1) * per * 16;
    if (*lo > j->nrows) *lo = j->nrows;
    if (*hi > j->nrows) *hi = j->nrows;
}

static void *worker(void *arg) {
    warg_t *wa = (warg_t *)arg;
    pool_t *p = wa->p;
    int id = wa->id, seen = 0;
    cpu_set_t set;
    CPU_ZERO(&set);
    CPU_SET(id, &set);
    pthread_setaffinity_np(pthread_self(), sizeof set, &set); /* best effort */
    for (;;) {
        while (atomic_load_explicit(&p->gen, memory_order_acquire) == seen) {
            if (atomic_load_explicit(&p->quit, memory_order_relaxed)) return NULL;
            _mm_pause();
        }
        seen++;
        int lo, hi;
        share(&p->job, p->nthreads, id, &lo, &hi);
        run_rows(p, &p->job, lo, hi);
        atomic_fetch_add_explicit(&p->done, 1, memory_order_release);
    }
}

pool_t *jlc_pool_create(int nthreads) {
    pool_t *p = (pool_t *)calloc(1, sizeof *p);
    if (!p) return NULL;
    if (nthreads < 1) nthreads = 1;
    p->nthreads = nthreads;
    __builtin_cpu_init();
    p->has_vnni = __builtin_cpu_supports("avxvnni");
    p->th = (pthread_t *)calloc((size_t)nthreads, sizeof(pthread_t));
    /* worker 0 is the calling thread */
    for (int i = 1; i < nthreads; i++) {
        warg_t *wa = (warg_t *)malloc(sizeof *wa);
        wa->p = p;
        wa->id = i;
        pthread_create(&p->th[i], NULL, worker, wa);
    }
    return p;
}

void jlc_pool_destroy(pool_t *p) {
    if (!p) return;
    atomic_store(&p->quit, 1);
    for (int i = 1; i < p->nthreads; i++) pthread_join(p->th[i], NULL);
    free(p->th);
    free(p->a); free(p->as); free(p->sum32); free(p->sum16);
    free(p);
}

int jlc_has_vnni(const pool_t *p) { return p->has_vnni; }
int jlc_threads(const pool_t *p) { return p->nthreads; }

/* The activation quantizer, vectorised (same values as the oracle's scalar form). */
__attribute__((target("avx2,fma"))) static void quantize(pool_t *p, const float *x, int k, int window) {
    if (k > p->cap_k) {
        free(p->a); free(p->as); free(p->sum32); free(p->sum16);
        p->a = (int8_t *)aligned_alloc(64, (size_t)k);
        p->as = (float *)malloc((size_t)(k / 32) * 4);
        p->sum32 = (float *)malloc((size_t)(k / 32) * 4);
        p->sum16 = (float *)malloc((size_t)(k / 16) * 4);
        p->cap_k = k;
    }
    const __m256 absm = _mm256_castsi256_ps(_mm256_set1_epi32(0x7FFFFFFF));
    const __m256 signm = _mm256_castsi256_ps(_mm256_set1_epi32((int)0x80000000u));
    const __m256 half = _mm256_castsi256_ps(_mm256_set1_epi32(0x3EFFFFFF)); /* 0.5 - 2^-25 */
    int per = window / 32 < 1 ? 1 : window / 32;
    for (int w0 = 0; w0 < k; w0 += per * 32) {
        int w1 = w0 + per * 32 > k ? k : w0 + per * 32;
        __m256 m = _mm256_setzero_ps();
        for (int i = w0; i < w1; i += 8) m = _mm256_max_ps(m, _mm256_and_ps(_mm256_loadu_ps(x + i), absm));
        float t[8];
        _mm256_storeu_ps(t, m);
        float amax = 0;
        for (int i = 0; i < 8; i++) amax = t[i] > amax ? t[i] : amax;
        float d = amax / 127.0f, inv = d != 0 ? 1.0f / d : 0.0f;
        __m256 vinv = _mm256_set1_ps(inv);
        for (int b = w0 / 32; b < w1 / 32; b++) {
            int sums[2] = {0, 0};
            for (int h = 0; h < 2; h++) {
                __m256i q[2];
                for (int v = 0; v < 2; v++) {
                    __m256 pv = _mm256_mul_ps(_mm256_loadu_ps(x + b * 32 + h * 16 + v * 8), vinv);
                    /* round half away from zero, exactly: add copysign(0.5 - 2^-25), truncate */
                    pv = _mm256_add_ps(pv, _mm256_or_ps(half, _mm256_and_ps(pv, signm)));
                    q[v] = _mm256_cvttps_epi32(pv);
                }
                int32_t qi[16];
                _mm256_storeu_si256((__m256i *)qi, q[0]);
                _mm256_storeu_si256((__m256i *)(qi + 8), q[1]);
                for (int i = 0; i < 16; i++) {
                    p->a[b * 32 + h * 16 + i] = (int8_t)qi[i];
                    sums[h] += qi[i];
                }
                p->sum16[b * 2 + h] = (float)sums[h];
            }
            p->as[b] = d;
            p->sum32[b] = (float)(sums[0] + sums[1]);
        }
    }
}

/* One decode matvec over packed planes, quantizing x first (NewInput + MatVecPacked,
 * engine/nn/perbyte_test.go:131-144).  nrows must be a multiple of 8. */
int jlc_matvec_packed(pool_t *p, float *out, int type, const uint32_t *qs, const uint32_t *d,
                      const uint32_t *sc, const float *x, int nrows, int k, int window) {
    if (nrows % 8 != 0 || k % 256 != 0) return -1;
    if (type != T_Q4_K && type != T_Q8_0 && type != T_Q6_K) return -1;
    quantize(p, x, k, window);
    job_t *j = &p->job;
    j->type = type; j->qs = qs; j->d = d; j->sc = sc;
    j->a = p->a; j->as = p->as; j->sum32 = p->sum32; j->sum16 = p->sum16;
    j->out = out; j->nrows = nrows; j->k = k;
    atomic_store_explicit(&p->done, 0, memory_order_relaxed);
    atomic_fetch_add_explicit(&p->gen, 1, memory_order_release);
    int lo, hi;
    share(j, p->nthreads, 0, &lo, &hi);
    run_rows(p, j, lo, hi);
    while (atomic_load_explicit(&p->done, memory_order_acquire) < p->nthreads - 1) _mm_pause();
    return 0;
}

/* Streams `n` distinct packed copies `reps` times and returns the best seconds per
 * call (3 warm calls first), the reference's protocol for a bandwidth-bound shape
 * (engine/nn/perbyte_test.go:184-292). */
/* Seconds per call: 3 warm calls, then `reps` timed passes (at most 32) of `sweeps` sweeps over
 * all the copies each; the MEDIAN pass (the reference's protocol, engine/nn/perbyte_test.go:131-144). */
double jlc_time_matvec(pool_t *p, float *out, int type, const uint32_t *const *qs,
                       const uint32_t *const *d, const uint32_t *const *sc, int ncopies,
                       const float *x, int nrows, int k, int window, int reps, int sweeps) {
    double pass[32];
    if (reps < 1 || reps > 32 || sweeps < 1) return -1;
    for (int i = 0; i < 3; i++)
        if (jlc_matvec_packed(p, out, type, qs[i % ncopies], d[i % ncopies], sc ? sc[i % ncopies] : NULL,
                              x, nrows, k, window)) return -1;
    for (int r = 0; r < reps; r++) {
        struct timespec t0, t1;
        clock_gettime(CLOCK_MONOTONIC, &t0);
        for (int s = 0; s < sweeps; s++)
            for (int i = 0; i < ncopies; i++)
                jlc_matvec_packed(p, out, type, qs[i], d[i], sc ? sc[i] : NULL, x, nrows, k, window);
        clock_gettime(CLOCK_MONOTONIC, &t1);
        pass[r] = ((t1.tv_sec - t0.tv_sec) + 1e-9 * (t1.tv_nsec - t0.tv_nsec)) / ((double)ncopies * sweeps);
    }
    for (int a = 1; a < reps; a++) {   /* insertion sort */
        double v = pass[a];
        int b = a - 1;
        for (; b >= 0 && pass[b] > v; b--) pass[b + 1] = pass[b];
        pass[b + 1] = v;
    }
    return reps & 1 ? pass[reps / 2] : 0.5 * (pass[reps / 2 - 1] + pass[reps / 2]);
}

/* Read-bandwidth wall of the host: every worker sums a private slice of `bytes`
 * (the role of dev/probe/cpu/membw.c).  Returns bytes per second. */
typedef struct { const uint8_t *p; size_t n; uint64_t sum; } bw_t;
__attribute__((target("avx2"))) static void *bw_worker(void *arg) {
    bw_t *b = (bw_t *)arg;
    __m256i acc = _mm256_setzero_si256();
    for (size_t i = 0; i + 32 <= b->n; i += 32)
        acc = _mm256_add_epi64(acc, _mm256_loadu_si256((const __m256i *)(b->p + i)));
    uint64_t t[4];
    _mm256_storeu_si256((__m256i *)t, acc);
    b->sum = t[0] + t[1] + t[2] + t[3];
    return NULL;
}
double jlc_membw(int nthreads, size_t bytes, int reps) {
    uint8_t *buf = (uint8_t *)aligned_alloc(64, bytes);
    if (!buf) return -1;
    memset(buf, 1, bytes);
    double best = 0;
    pthread_t *th = (pthread_t *)calloc((size_t)nthreads, sizeof(pthread_t));
    bw_t *bw = (bw_t *)calloc((size_t)nthreads, sizeof(bw_t));
    for (int r = 0; r < reps; r++) {
        struct timespec t0, t1;
        clock_gettime(CLOCK_MONOTONIC, &t0);
        size_t per = bytes / (size_t)nthreads / 32 * 32;
        for (int i = 0; i < nthreads; i++) {
            bw[i].p = buf + per * (size_t)i;
            bw[i].n = per;
            pthread_create(&th[i], NULL, bw_worker, &bw[i]);
        }
        for (int i = 0; i < nthreads; i++) pthread_join(th[i], NULL);
        clock_gettime(CLOCK_MONOTONIC, &t1);
        double s = (t1.tv_sec - t0.tv_sec) + 1e-9 * (t1.tv_nsec - t0.tv_nsec);
        double rate = (double)(per * (size_t)nthreads) / s;
        if (rate > best) best = rate;
    }
    free(th); free(bw); free(buf);
    return best;
}
