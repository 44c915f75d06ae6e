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
 *   prefill GEMM           jit/cpu/packedgemm.go:37-75 (EmitPackedMatMulStationary, the
 *                          VNNI form that keeps the float epilogue): a sub-block of eight
 *                          rows is decoded into eight registers once and dotted against
 *                          every token of the call, the tokens innermost; work items are
 *                          (16 rows, up to 64 tokens) handed to the workers one at a time,
 *                          outputs accumulated in a scratch whose token rows are a cache
 *                          line longer than the matrix is tall (engine/nn/packedmm.go:424-478)
 *   mixture block          engine/model/moe.go:697-761 (moeBatchExpert): expert by expert in
 *                          ascending id, the rows that chose it gathered, gate and up
 *                          through the GEMM, silu(g) * u, down through the GEMM, the
 *                          residual add in that order
 *
 * Formats: Q4_K, Q8_0, Q6_K (the decode configurations); the GEMM and the mixture block
 * Q4_K.  Nothing in the product library links or calls this file.
 */
#define _GNU_SOURCE
#include <immintrin.h>
#include <pthread.h>
#include <sched.h>
#include <stdatomic.h>
#include <stdint.h>
#include <math.h>
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

/* A prefill GEMM over Q4_K planes: out [ntok][nrows] += x W^T on quantized activations. */
#define GEMM_PAD 64 /* bytes after each token's row of every per-token stream (cpu.GEMMPad) */
typedef struct {
    const uint32_t *qs, *d, *sc;
    int row0, stride;     /* the matrix is rows row0.. of planes `stride` rows long (an expert's sheet) */
    const float *x;       /* [ntok][k], quantized by the workers first */
    int8_t *a;            /* [ntok][k + GEMM_PAD] */
    float *as, *sum32;    /* [ntok][k/32 + GEMM_PAD/4] */
    float *mout;          /* [ntok][nrows + GEMM_PAD/4] */
    int nrows, k, ntok, window, tok_block;
} gemm_t;

enum { JOB_ROWS = 0, JOB_QUANT = 1, JOB_GEMM = 2 };

typedef struct pool {
    int nthreads;
    pthread_t *th;
    _Atomic int gen, done, quit;
    int kind;
    _Atomic int next;     /* the next work item of a JOB_QUANT / JOB_GEMM region */
    job_t job;
    gemm_t gemm;
    int has_vnni;
    /* quantized activation scratch */
    int8_t *a;
    float *as, *sum32, *sum16;
    int cap_k;
    /* prefill scratch, grown on demand */
    int8_t *ga;
    float *gas, *gsum, *gout;
    size_t ga_cap, gs_cap, go_cap;
    /* mixture block scratch */
    float *mx, *mg, *mu, *my;
    size_t mx_cap, mg_cap;
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

static void run_region(pool_t *p, int id);

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
        run_region(p, id);
        atomic_fetch_add_explicit(&p->done, 1, memory_order_release);
    }
}

/* One region on every worker (the caller is worker 0); returns when all have finished. */
static void pool_run(pool_t *p, int kind) {
    p->kind = kind;
    atomic_store_explicit(&p->next, 0, memory_order_relaxed);
    atomic_store_explicit(&p->done, 0, memory_order_relaxed);
    atomic_fetch_add_explicit(&p->gen, 1, memory_order_release);
    run_region(p, 0);
    while (atomic_load_explicit(&p->done, memory_order_acquire) < p->nthreads - 1) _mm_pause();
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
    free(p->ga); free(p->gas); free(p->gsum); free(p->gout);
    free(p->mx); free(p->mg); free(p->mu); free(p->my);
    free(p);
}

int jlc_has_vnni(const pool_t *p) { return p->has_vnni; }
int jlc_threads(const pool_t *p) { return p->nthreads; }

/* The activation quantizer, vectorised (same values as the oracle's scalar form). */
__attribute__((target("avx2,fma"))) static void quantize_into(const float *x, int k, int window, int8_t *qa,
                                                              float *qas, float *qsum32, float *qsum16);

static void quantize(pool_t *p, const float *x, int k, int window) {
    if (k > p->cap_k) {
        free(p->a); free(p->as); free(p->sum32); free(p->sum16);
        p->a = (int8_t *)aligned_alloc(64, (size_t)k);
        p->as = (float *)malloc((size_t)(k / 32) * 4);
        p->sum32 = (float *)malloc((size_t)(k / 32) * 4);
        p->sum16 = (float *)malloc((size_t)(k / 16) * 4);
        p->cap_k = k;
    }
    quantize_into(x, k, window, p->a, p->as, p->sum32, p->sum16);
}

/* qsum16 may be null. */
__attribute__((target("avx2,fma"))) static void quantize_into(const float *x, int k, int window, int8_t *qa,
                                                              float *qas, float *qsum32, float *qsum16) {
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
                    qa[b * 32 + h * 16 + i] = (int8_t)qi[i];
                    sums[h] += qi[i];
                }
                if (qsum16) qsum16[b * 2 + h] = (float)sums[h];
            }
            qas[b] = d;
            qsum32[b] = (float)(sums[0] + sums[1]);
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
    pool_run(p, JOB_ROWS);
    return 0;
}

/* ------------------------------------------------------------ prefill GEMM (Q4_K) */

/* One work item: rows [r0, r1) (multiples of 8) against tokens [t0, t1).  For every group of
 * eight rows and every sub-block: the row group's scale d*sc and bias dmin*m, the sub-block's
 * four words split into eight registers of bytes (low field, high field), then the tokens:
 * eight VPDPBUSD against broadcast activation words, and the fused kernel's float epilogue
 * into the token's eight outputs. */
#define GEMM_ITEM(DP, TARGET)                                                                             \
    __attribute__((target(TARGET))) static void gemm_item_##DP(const gemm_t *g, int r0, int r1, int t0,    \
                                                               int t1) {                                  \
        const int nsub = g->k / 32, st = g->stride;                                                       \
        const size_t astr = (size_t)g->k + GEMM_PAD, sstr = (size_t)(g->k / 32) + GEMM_PAD / 4;           \
        const size_t ostr = (size_t)g->nrows + GEMM_PAD / 4;                                              \
        const __m256i m4 = _mm256_set1_epi32(0x0F0F0F0F);                                                 \
        for (int r = r0; r < r1; r += 8) {                                                                \
            const size_t pr = (size_t)g->row0 + r;                                                        \
            for (int si = 0; si < nsub; si++) {                                                           \
                const int sup = si >> 3, s = si & 7;                                                      \
                __m256i W[8];                                                                             \
                for (int w = 0; w < 4; w++) {                                                             \
                    __m256i pay = _mm256_loadu_si256((const __m256i *)(g->qs + ((size_t)si * 4 + w) * st + pr)); \
                    W[w] = _mm256_and_si256(pay, m4);                                                     \
                    W[4 + w] = _mm256_and_si256(_mm256_srli_epi32(pay, 4), m4);                           \
                }                                                                                         \
                __m256i dw = _mm256_loadu_si256((const __m256i *)(g->d + (size_t)sup * st + pr));         \
                __m256i dlo = _mm256_and_si256(dw, _mm256_set1_epi32(0xFFFF));                            \
                __m256i dhi = _mm256_srli_epi32(dw, 16);                                                  \
                __m256 d = _mm256_cvtph_ps(_mm256_castsi256_si128(_mm256_permute4x64_epi64(               \
                    _mm256_packus_epi32(dlo, dlo), 0xD8)));                                               \
                __m256 dmin = _mm256_cvtph_ps(_mm256_castsi256_si128(_mm256_permute4x64_epi64(            \
                    _mm256_packus_epi32(dhi, dhi), 0xD8)));                                               \
                __m256i ws[3], scv, mv;                                                                   \
                for (int w = 0; w < 3; w++)                                                               \
                    ws[w] = _mm256_loadu_si256((const __m256i *)(g->sc + ((size_t)sup * 3 + w) * st + pr)); \
                SC_FIELD(ws, s, 0, scv);                                                                  \
                SC_FIELD(ws, s, 1, mv);                                                                   \
                const __m256 dsc = _mm256_mul_ps(d, _mm256_cvtepi32_ps(scv));                             \
                const __m256 dm = _mm256_mul_ps(dmin, _mm256_cvtepi32_ps(mv));                            \
                for (int t = t0; t < t1; t++) {                                                           \
                    const uint32_t *a32 = (const uint32_t *)(g->a + (size_t)t * astr + (size_t)si * 32);  \
                    const float da = g->as[(size_t)t * sstr + si];                                        \
                    __m256i iacc = _mm256_setzero_si256();                                                \
                    for (int w = 0; w < 4; w++) {                                                         \
                        iacc = dp_##DP(iacc, W[w], _mm256_set1_epi32((int)a32[w]));                       \
                        iacc = dp_##DP(iacc, W[4 + w], _mm256_set1_epi32((int)a32[4 + w]));               \
                    }                                                                                     \
                    float *op = g->mout + (size_t)t * ostr + r;                                           \
                    __m256 o = _mm256_loadu_ps(op);                                                       \
                    o = _mm256_fmadd_ps(_mm256_cvtepi32_ps(iacc), _mm256_mul_ps(dsc, _mm256_set1_ps(da)), o); \
                    o = _mm256_fnmadd_ps(dm, _mm256_set1_ps(g->sum32[(size_t)t * sstr + si] * da), o);    \
                    _mm256_storeu_ps(op, o);                                                              \
                }                                                                                         \
            }                                                                                             \
        }                                                                                                 \
    }
GEMM_ITEM(vnni, "avx2,avxvnni,fma,f16c")
GEMM_ITEM(vex, "avx2,fma,f16c")

static void run_region(pool_t *p, int id) {
    if (p->kind == JOB_ROWS) {
        int lo, hi;
        share(&p->job, p->nthreads, id, &lo, &hi);
        run_rows(p, &p->job, lo, hi);
        return;
    }
    const gemm_t *g = &p->gemm;
    if (p->kind == JOB_QUANT) {
        const size_t astr = (size_t)g->k + GEMM_PAD, sstr = (size_t)(g->k / 32) + GEMM_PAD / 4;
        for (;;) {
            int t = atomic_fetch_add_explicit(&p->next, 1, memory_order_relaxed);
            if (t >= g->ntok) break;
            quantize_into(g->x + (size_t)t * g->k, g->k, g->window, g->a + (size_t)t * astr, g->as + (size_t)t * sstr,
                          g->sum32 + (size_t)t * sstr, NULL);
            memset(g->mout + (size_t)t * ((size_t)g->nrows + GEMM_PAD / 4), 0, (size_t)g->nrows * 4);
        }
        return;
    }
    /* JOB_GEMM: items are (block of 16 rows, block of tok_block tokens), one at a time */
    const int nrc = (g->nrows + 15) / 16, ntt = (g->ntok + g->tok_block - 1) / g->tok_block;
    for (;;) {
        int it = atomic_fetch_add_explicit(&p->next, 1, memory_order_relaxed);
        if (it >= nrc * ntt) break;
        const int r0 = (it / ntt) * 16, t0 = (it % ntt) * g->tok_block;
        const int r1 = r0 + 16 < g->nrows ? r0 + 16 : g->nrows;
        const int t1 = t0 + g->tok_block < g->ntok ? t0 + g->tok_block : g->ntok;
        if (p->has_vnni) gemm_item_vnni(g, r0, r1, t0, t1);
        else gemm_item_vex(g, r0, r1, t0, t1);
    }
}

static int gemm_grow(pool_t *p, int ntok, int nrows, int k) {
    const size_t na = (size_t)ntok * ((size_t)k + GEMM_PAD);
    const size_t ns = (size_t)ntok * ((size_t)(k / 32) + GEMM_PAD / 4);
    const size_t no = (size_t)ntok * ((size_t)nrows + GEMM_PAD / 4);
    if (na > p->ga_cap) { free(p->ga); p->ga = (int8_t *)aligned_alloc(64, (na + 63) & ~(size_t)63); p->ga_cap = na; }
    if (ns > p->gs_cap) {
        free(p->gas); free(p->gsum);
        p->gas = (float *)malloc(ns * 4); p->gsum = (float *)malloc(ns * 4); p->gs_cap = ns;
    }
    if (no > p->go_cap) { free(p->gout); p->gout = (float *)malloc(no * 4); p->go_cap = no; }
    return p->ga && p->gas && p->gsum && p->gout ? 0 : -1;
}

/* out [ntok][nrows] = x [ntok][k] W^T over rows row0.. of Q4_K planes `stride` rows long: the
 * activation quantizer over every token, the weight-stationary GEMM into the padded scratch,
 * the copy out (engine/nn/packedmm.go:424-478).  nrows a multiple of 8. */
int jlc_matmul_packed(pool_t *p, float *out, int type, const uint32_t *qs, const uint32_t *d, const uint32_t *sc,
                      int row0, int stride, const float *x, int nrows, int k, int ntok, int window) {
    if (type != T_Q4_K || nrows % 8 != 0 || k % 256 != 0 || ntok < 1) return -1;
    if (gemm_grow(p, ntok, nrows, k)) return -1;
    gemm_t *g = &p->gemm;
    g->qs = qs; g->d = d; g->sc = sc; g->row0 = row0; g->stride = stride;
    g->x = x; g->a = p->ga; g->as = p->gas; g->sum32 = p->gsum; g->mout = p->gout;
    g->nrows = nrows; g->k = k; g->ntok = ntok; g->window = window;
    /* tokens a call: min(64, max(8, 4 Mi MACs / (16 rows * k), rounded down to eight)) */
    int T = (4 << 20) / (16 * k) / 8 * 8;
    T = T < 8 ? 8 : T > 64 ? 64 : T;
    g->tok_block = T < ntok ? T : ntok;
    pool_run(p, JOB_QUANT);
    pool_run(p, JOB_GEMM);
    const size_t ostr = (size_t)nrows + GEMM_PAD / 4;
    for (int t = 0; t < ntok; t++) memcpy(out + (size_t)t * nrows, g->mout + (size_t)t * ostr, (size_t)nrows * 4);
    return 0;
}

/* Seconds per call: 3 warm calls, then the median of `reps` (<= 32) timed calls. */
double jlc_time_matmul(pool_t *p, float *out, int type, const uint32_t *qs, const uint32_t *d, const uint32_t *sc,
                       const float *x, int nrows, int k, int ntok, int window, int reps) {
    double pass[32];
    if (reps < 1 || reps > 32) return -1;
    for (int i = 0; i < 3; i++)
        if (jlc_matmul_packed(p, out, type, qs, d, sc, 0, nrows, x, nrows, k, ntok, window)) return -1;
    for (int r = 0; r < reps; r++) {
        struct timespec t0, t1;
        clock_gettime(CLOCK_MONOTONIC, &t0);
        jlc_matmul_packed(p, out, type, qs, d, sc, 0, nrows, x, nrows, k, ntok, window);
        clock_gettime(CLOCK_MONOTONIC, &t1);
        pass[r] = (t1.tv_sec - t0.tv_sec) + 1e-9 * (t1.tv_nsec - t0.tv_nsec);
    }
    for (int a = 1; a < reps; a++) {
        double v = pass[a];
        int b = a - 1;
        for (; b >= 0 && pass[b] > v; b--) pass[b + 1] = pass[b];
        pass[b + 1] = v;
    }
    return reps & 1 ? pass[reps / 2] : 0.5 * (pass[reps / 2 - 1] + pass[reps / 2]);
}

/* ------------------------------------------------------------ mixture block (Q4_K) */

/* resid [rows][n_embd] += the routed feed-forward block: expert by expert in ascending id, the
 * rows that chose it gathered (row order), gate and up through the GEMM, silu(g) * u, down
 * through the GEMM, resid[row] += weight * y (engine/model/moe.go:697-761).  Banks are plane
 * sets of n_expert * rows rows, an expert's sheet its row range.  sel [rows][sel_stride],
 * wt [rows][k_used].  n_ffn and n_embd multiples of 256. */
int jlc_moe_block(pool_t *p, float *resid, const uint32_t *const *gate, const uint32_t *const *up,
                  const uint32_t *const *down, const float *x, const uint32_t *sel, int sel_stride, const float *wt,
                  int rows, int k_used, int n_expert, int n_ffn, int n_embd, int window) {
    if (n_ffn % 256 || n_embd % 256 || rows < 1) return -1;
    const size_t nx = (size_t)rows * n_embd, ng = (size_t)rows * n_ffn;
    if (nx > p->mx_cap) {
        free(p->mx); free(p->my);
        p->mx = (float *)malloc(nx * 4); p->my = (float *)malloc(nx * 4); p->mx_cap = nx;
    }
    if (ng > p->mg_cap) {
        free(p->mg); free(p->mu);
        p->mg = (float *)malloc(ng * 4); p->mu = (float *)malloc(ng * 4); p->mg_cap = ng;
    }
    if (!p->mx || !p->my || !p->mg || !p->mu) return -1;
    int *row_of = (int *)malloc((size_t)rows * sizeof(int));
    float *w_of = (float *)malloc((size_t)rows * sizeof(float));
    if (!row_of || !w_of) { free(row_of); free(w_of); return -1; }
    int rc = 0;
    for (int e = 0; e < n_expert && !rc; e++) {
        int m = 0;
        for (int i = 0; i < rows; i++)
            for (int j = 0; j < k_used; j++)
                if (sel[(size_t)i * sel_stride + j] == (uint32_t)e) {
                    row_of[m] = i;
                    w_of[m] = wt[(size_t)i * k_used + j];
                    m++;
                    break;
                }
        if (!m) continue;
        for (int r = 0; r < m; r++) memcpy(p->mx + (size_t)r * n_embd, x + (size_t)row_of[r] * n_embd, (size_t)n_embd * 4);
        rc = jlc_matmul_packed(p, p->mg, T_Q4_K, gate[0], gate[1], gate[2], e * n_ffn, n_expert * n_ffn, p->mx, n_ffn,
                               n_embd, m, window);
        if (!rc)
            rc = jlc_matmul_packed(p, p->mu, T_Q4_K, up[0], up[1], up[2], e * n_ffn, n_expert * n_ffn, p->mx, n_ffn,
                                   n_embd, m, window);
        if (rc) break;
        for (size_t i = 0; i < (size_t)m * n_ffn; i++) {
            const float g = p->mg[i];
            p->mg[i] = g / (1.0f + expf(-g)) * p->mu[i];
        }
        rc = jlc_matmul_packed(p, p->my, T_Q4_K, down[0], down[1], down[2], e * n_embd, n_expert * n_embd, p->mg,
                               n_embd, n_ffn, m, window);
        if (rc) break;
        for (int r = 0; r < m; r++) {
            float *dst = resid + (size_t)row_of[r] * n_embd;
            const float *y = p->my + (size_t)r * n_embd;
            for (int c = 0; c < n_embd; c++) dst[c] += w_of[r] * y[c];
        }
    }
    free(row_of); free(w_of);
    return rc;
}

/* Seconds per block: one warm call, then the median of `reps` (<= 32) timed calls (the
 * residual is zeroed before each). */
double jlc_time_moe_block(pool_t *p, float *resid, const uint32_t *const *gate, const uint32_t *const *up,
                          const uint32_t *const *down, const float *x, const uint32_t *sel, int sel_stride,
                          const float *wt, int rows, int k_used, int n_expert, int n_ffn, int n_embd, int window,
                          int reps) {
    double pass[32];
    if (reps < 1 || reps > 32) return -1;
    memset(resid, 0, (size_t)rows * n_embd * 4);
    if (jlc_moe_block(p, resid, gate, up, down, x, sel, sel_stride, wt, rows, k_used, n_expert, n_ffn, n_embd, window))
        return -1;
    for (int r = 0; r < reps; r++) {
        struct timespec t0, t1;
        memset(resid, 0, (size_t)rows * n_embd * 4);
        clock_gettime(CLOCK_MONOTONIC, &t0);
        jlc_moe_block(p, resid, gate, up, down, x, sel, sel_stride, wt, rows, k_used, n_expert, n_ffn, n_embd, window);
        clock_gettime(CLOCK_MONOTONIC, &t1);
        pass[r] = (t1.tv_sec - t0.tv_sec) + 1e-9 * (t1.tv_nsec - t0.tv_nsec);
    }
    for (int a = 1; a < reps; a++) {
        double v = pass[a];
        int b = a - 1;
        for (; b >= 0 && pass[b] > v; b--) pass[b + 1] = pass[b];
        pass[b + 1] = v;
    }
    return reps & 1 ? pass[reps / 2] : 0.5 * (pass[reps / 2 - 1] + pass[reps / 2]);
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
