/* AVX2/FMA build of the CPU oracle: the reference's x86_64 row kernels in
 * intrinsics, spread over a persistent worker pool with the reference's
 * row-chunk schedule.  TEST INFRASTRUCTURE (see joshua_oracle.h); this is the
 * timed CPU baseline.  Build with -mavx2 -mfma -mf16c -ffp-contract=off. */
#include "joshua_oracle.h"

#include <immintrin.h>
#include <pthread.h>
#include <stdatomic.h>
#include <stdlib.h>
#include <string.h>
#include <unistd.h>

/* from joshua_oracle.c */
int orc_fail(const char *fmt, ...);
int orc_validate(uint32_t type, size_t m, size_t k, size_t n, size_t lhs_len, size_t nbytes,
                 size_t dst_len, size_t *bpr);
void orc_q4k_scale_min(const uint8_t *s, int j, uint8_t *sc, uint8_t *mn);
void orc_iq2xxs_grid(int code, uint8_t out[8]);
uint8_t orc_iq2xxs_signs(unsigned i);
float orc_e8m0(uint8_t e, int *ok);
float orc_f16_to_f32(uint16_t h);

int orc_have_avx2(void) {
    return __builtin_cpu_supports("avx2") && __builtin_cpu_supports("fma") &&
           __builtin_cpu_supports("f16c");
}

int orc_default_threads(void) {
    long n = sysconf(_SC_NPROCESSORS_ONLN);
    return n < 1 ? 1 : (int)n;
}

/* ---- worker pool with the reference's chunking -------------------------- *
 * reference: src/simd.rs:128-145 — serial when threads <= 1 or n < 8, else
 * contiguous chunks of max(n/(threads*4), 1) rows handed to idle workers.   */

typedef void (*rows_fn)(void *ctx, size_t row_begin, size_t row_end);

typedef struct {
    pthread_mutex_t mu;
    pthread_cond_t start, done;
    pthread_t *tids;
    int nthreads; /* helpers, excluding the caller */
    unsigned long generation;
    int running, shutdown;
    rows_fn fn;
    void *ctx;
    size_t n, chunk;
    atomic_size_t next;
} pool_t;

static pool_t g_pool;
static pthread_mutex_t g_pool_guard = PTHREAD_MUTEX_INITIALIZER;

static void pool_drain(pool_t *p) {
    for (;;) {
        size_t c = atomic_fetch_add(&p->next, 1);
        size_t b = c * p->chunk;
        if (b >= p->n) break;
        size_t e = b + p->chunk;
        if (e > p->n) e = p->n;
        p->fn(p->ctx, b, e);
    }
}

static void *pool_main(void *arg) {
    pool_t *p = (pool_t *)arg;
    unsigned long seen = 0;
    pthread_mutex_lock(&p->mu);
    for (;;) {
        while (!p->shutdown && p->generation == seen) pthread_cond_wait(&p->start, &p->mu);
        if (p->shutdown) break;
        seen = p->generation;
        pthread_mutex_unlock(&p->mu);
        pool_drain(p);
        pthread_mutex_lock(&p->mu);
        if (--p->running == 0) pthread_cond_signal(&p->done);
    }
    pthread_mutex_unlock(&p->mu);
    return NULL;
}

static void pool_resize(pool_t *p, int helpers) {
    if (p->tids && p->nthreads == helpers) return;
    if (p->tids) {
        pthread_mutex_lock(&p->mu);
        p->shutdown = 1;
        pthread_cond_broadcast(&p->start);
        pthread_mutex_unlock(&p->mu);
        for (int i = 0; i < p->nthreads; i++) pthread_join(p->tids[i], NULL);
        free(p->tids);
        p->tids = NULL;
    } else {
        pthread_mutex_init(&p->mu, NULL);
        pthread_cond_init(&p->start, NULL);
        pthread_cond_init(&p->done, NULL);
    }
    p->shutdown = 0;
    p->nthreads = helpers;
    p->tids = (pthread_t *)calloc((size_t)(helpers > 0 ? helpers : 1), sizeof(pthread_t));
    for (int i = 0; i < helpers; i++) pthread_create(&p->tids[i], NULL, pool_main, p);
}

static void run_chunks(int threads, size_t n, rows_fn fn, void *ctx) {
    if (threads <= 1 || n < 8) {
        fn(ctx, 0, n);
        return;
    }
    pthread_mutex_lock(&g_pool_guard);
    pool_t *p = &g_pool;
    pool_resize(p, threads - 1);
    size_t chunk = n / ((size_t)threads * 4);
    if (chunk < 1) chunk = 1;
    pthread_mutex_lock(&p->mu);
    p->fn = fn;
    p->ctx = ctx;
    p->n = n;
    p->chunk = chunk;
    atomic_store(&p->next, 0);
    p->running = p->nthreads;
    p->generation++;
    pthread_cond_broadcast(&p->start);
    pthread_mutex_unlock(&p->mu);
    pool_drain(p);
    pthread_mutex_lock(&p->mu);
    while (p->running > 0) pthread_cond_wait(&p->done, &p->mu);
    pthread_mutex_unlock(&p->mu);
    pthread_mutex_unlock(&g_pool_guard);
}

/* ---- row kernels --------------------------------------------------------- */

#define MTILE 4

typedef struct {
    uint32_t type;
    size_t m, k, n, bpr;
    const float *lhs;
    const uint8_t *blocks;
    float *dst;
} job_t;

/* reference: src/simd.rs:198-206 */
static inline float hsum256(__m256 v) {
    __m128 hi = _mm256_extractf128_ps(v, 1);
    __m128 lo = _mm256_castps256_ps128(v);
    __m128 s = _mm_add_ps(lo, hi);
    s = _mm_add_ps(s, _mm_movehl_ps(s, s));
    s = _mm_add_ps(s, _mm_shuffle_ps(s, s, 1));
    return _mm_cvtss_f32(s);
}

static inline float f16_ld(const uint8_t *p) {
    uint16_t h;
    memcpy(&h, p, 2);
    return _cvtsh_ss(h);
}

static inline __m256 cvt8_i8(__m128i v) { return _mm256_cvtepi32_ps(_mm256_cvtepi8_epi32(v)); }
static inline __m256 cvt8_u8(__m128i v) { return _mm256_cvtepi32_ps(_mm256_cvtepu8_epi32(v)); }

/* reference: src/kquant_dot.rs:268-319 */
static void row_q8_0(const job_t *j, size_t row) {
    const uint8_t *rb = j->blocks + row * j->bpr * 34;
    for (size_t m0 = 0; m0 < j->m; m0 += MTILE) {
        size_t mcnt = j->m - m0 < MTILE ? j->m - m0 : MTILE;
        __m256 acc[MTILE];
        for (int i = 0; i < MTILE; i++) acc[i] = _mm256_setzero_ps();
        for (size_t b = 0; b < j->bpr; b++) {
            const uint8_t *blk = rb + b * 34;
            __m256 d4 = _mm256_set1_ps(f16_ld(blk));
            __m128i lo = _mm_loadu_si128((const __m128i *)(blk + 2));
            __m128i hi = _mm_loadu_si128((const __m128i *)(blk + 18));
            __m256 w0 = _mm256_mul_ps(cvt8_i8(lo), d4);
            __m256 w1 = _mm256_mul_ps(cvt8_i8(_mm_srli_si128(lo, 8)), d4);
            __m256 w2 = _mm256_mul_ps(cvt8_i8(hi), d4);
            __m256 w3 = _mm256_mul_ps(cvt8_i8(_mm_srli_si128(hi, 8)), d4);
            for (size_t i = 0; i < mcnt; i++) {
                const float *a = j->lhs + (m0 + i) * j->k + b * 32;
                acc[i] = _mm256_fmadd_ps(_mm256_loadu_ps(a), w0, acc[i]);
                acc[i] = _mm256_fmadd_ps(_mm256_loadu_ps(a + 8), w1, acc[i]);
                acc[i] = _mm256_fmadd_ps(_mm256_loadu_ps(a + 16), w2, acc[i]);
                acc[i] = _mm256_fmadd_ps(_mm256_loadu_ps(a + 24), w3, acc[i]);
            }
        }
        for (size_t i = 0; i < mcnt; i++) j->dst[(m0 + i) * j->n + row] = hsum256(acc[i]);
    }
}

/* reference: src/kquant_dot.rs:326-400 */
static void row_q2_k(const job_t *j, size_t row) {
    const uint8_t *rb = j->blocks + row * j->bpr * 84;
    const __m256i m3 = _mm256_set1_epi8(3);
    for (size_t m0 = 0; m0 < j->m; m0 += MTILE) {
        size_t mcnt = j->m - m0 < MTILE ? j->m - m0 : MTILE;
        __m256 acc[MTILE];
        for (int i = 0; i < MTILE; i++) acc[i] = _mm256_setzero_ps();
        for (size_t b = 0; b < j->bpr; b++) {
            const uint8_t *blk = rb + b * 84;
            float d = f16_ld(blk + 80), dmin = f16_ld(blk + 82);
            for (int sg = 0; sg < 2; sg++) {
                __m256i x = _mm256_loadu_si256((const __m256i *)(blk + 16 + sg * 32));
                __m256i xf[4] = {_mm256_and_si256(x, m3),
                                 _mm256_and_si256(_mm256_srli_epi16(x, 2), m3),
                                 _mm256_and_si256(_mm256_srli_epi16(x, 4), m3),
                                 _mm256_and_si256(_mm256_srli_epi16(x, 6), m3)};
                for (int g = 0; g < 8; g++) {
                    uint8_t sc = blk[sg * 8 + g];
                    __m256 d1 = _mm256_set1_ps(d * (float)(sc & 0xF));
                    __m256 m1 = _mm256_set1_ps(dmin * (float)(sc >> 4));
                    __m256i xv = xf[g / 2];
                    __m128i bytes = (g % 2 == 0) ? _mm256_castsi256_si128(xv)
                                                 : _mm256_extracti128_si256(xv, 1);
                    __m256 w0 = _mm256_fmsub_ps(cvt8_u8(bytes), d1, m1);
                    __m256 w1 = _mm256_fmsub_ps(cvt8_u8(_mm_srli_si128(bytes, 8)), d1, m1);
                    size_t a = b * 256 + (size_t)sg * 128 + 16 * (size_t)g;
                    for (size_t i = 0; i < mcnt; i++) {
                        const float *p = j->lhs + (m0 + i) * j->k + a;
                        acc[i] = _mm256_fmadd_ps(_mm256_loadu_ps(p), w0, acc[i]);
                        acc[i] = _mm256_fmadd_ps(_mm256_loadu_ps(p + 8), w1, acc[i]);
                    }
                }
            }
        }
        for (size_t i = 0; i < mcnt; i++) j->dst[(m0 + i) * j->n + row] = hsum256(acc[i]);
    }
}

/* reference: src/kquant_dot.rs:407-483 */
static void row_q4_k(const job_t *j, size_t row) {
    const uint8_t *rb = j->blocks + row * j->bpr * 144;
    const __m256i mf = _mm256_set1_epi8(0x0F);
    for (size_t m0 = 0; m0 < j->m; m0 += MTILE) {
        size_t mcnt = j->m - m0 < MTILE ? j->m - m0 : MTILE;
        __m256 acc[MTILE];
        for (int i = 0; i < MTILE; i++) acc[i] = _mm256_setzero_ps();
        for (size_t b = 0; b < j->bpr; b++) {
            const uint8_t *blk = rb + b * 144;
            float d = f16_ld(blk), dmin = f16_ld(blk + 2);
            for (int c = 0; c < 4; c++) {
                __m256i x = _mm256_loadu_si256((const __m256i *)(blk + 16 + c * 32));
                __m256i x_lo = _mm256_and_si256(x, mf);
                __m256i x_hi = _mm256_and_si256(_mm256_srli_epi16(x, 4), mf);
                for (int r = 0; r < 2; r++) {
                    __m256i xv = r == 0 ? x_lo : x_hi;
                    uint8_t sc, mn;
                    orc_q4k_scale_min(blk + 4, 2 * c + r, &sc, &mn);
                    __m256 d1 = _mm256_set1_ps(d * (float)sc);
                    __m256 m1 = _mm256_set1_ps(dmin * (float)mn);
                    __m128i low = _mm256_castsi256_si128(xv);
                    __m128i high = _mm256_extracti128_si256(xv, 1);
                    __m256 w0 = _mm256_fmsub_ps(cvt8_u8(low), d1, m1);
                    __m256 w1 = _mm256_fmsub_ps(cvt8_u8(_mm_srli_si128(low, 8)), d1, m1);
                    __m256 w2 = _mm256_fmsub_ps(cvt8_u8(high), d1, m1);
                    __m256 w3 = _mm256_fmsub_ps(cvt8_u8(_mm_srli_si128(high, 8)), d1, m1);
                    size_t a = b * 256 + 64 * (size_t)c + 32 * (size_t)r;
                    for (size_t i = 0; i < mcnt; i++) {
                        const float *p = j->lhs + (m0 + i) * j->k + a;
                        acc[i] = _mm256_fmadd_ps(_mm256_loadu_ps(p), w0, acc[i]);
                        acc[i] = _mm256_fmadd_ps(_mm256_loadu_ps(p + 8), w1, acc[i]);
                        acc[i] = _mm256_fmadd_ps(_mm256_loadu_ps(p + 16), w2, acc[i]);
                        acc[i] = _mm256_fmadd_ps(_mm256_loadu_ps(p + 24), w3, acc[i]);
                    }
                }
            }
        }
        for (size_t i = 0; i < mcnt; i++) j->dst[(m0 + i) * j->n + row] = hsum256(acc[i]);
    }
}

/* f32 lookup tables the reference builds at compile time
 * (reference: src/iq2xxs.rs:272-315). */
static float g_grid_f32[256][8] __attribute__((aligned(32)));
static float g_signs_f32[128][8] __attribute__((aligned(32)));
static pthread_once_t g_tables_once = PTHREAD_ONCE_INIT;

static void build_tables(void) {
    for (int i = 0; i < 256; i++) {
        uint8_t g[8];
        orc_iq2xxs_grid(i, g);
        for (int jj = 0; jj < 8; jj++) g_grid_f32[i][jj] = (float)g[jj];
    }
    for (unsigned i = 0; i < 128; i++) {
        uint8_t s = orc_iq2xxs_signs(i);
        for (int jj = 0; jj < 8; jj++) g_signs_f32[i][jj] = (s & (1u << jj)) ? -1.0f : 1.0f;
    }
}

/* reference: src/iq2xxs.rs:331-391 */
static void row_iq2_xxs(const job_t *j, size_t row) {
    const uint8_t *rb = j->blocks + row * j->bpr * 66;
    for (size_t m0 = 0; m0 < j->m; m0 += MTILE) {
        size_t mcnt = j->m - m0 < MTILE ? j->m - m0 : MTILE;
        __m256 acc[MTILE];
        for (int i = 0; i < MTILE; i++) acc[i] = _mm256_setzero_ps();
        for (size_t b = 0; b < j->bpr; b++) {
            const uint8_t *blk = rb + b * 66;
            float d = f16_ld(blk);
            for (int ib32 = 0; ib32 < 8; ib32++) {
                uint32_t lo, hi;
                memcpy(&lo, blk + 2 + 8 * ib32, 4);
                memcpy(&hi, blk + 2 + 8 * ib32 + 4, 4);
                __m256 dbv = _mm256_set1_ps(d * (0.5f + (float)(hi >> 28)) * 0.25f);
                for (int l = 0; l < 4; l++) {
                    unsigned code = (lo >> (8 * l)) & 0xFF;
                    unsigned si = (hi >> (7 * l)) & 0x7F;
                    __m256 g = _mm256_load_ps(g_grid_f32[code]);
                    __m256 s = _mm256_load_ps(g_signs_f32[si]);
                    __m256 v = _mm256_mul_ps(_mm256_mul_ps(g, s), dbv);
                    size_t c = b * 256 + (size_t)ib32 * 32 + (size_t)l * 8;
                    for (size_t i = 0; i < mcnt; i++) {
                        __m256 a = _mm256_loadu_ps(j->lhs + (m0 + i) * j->k + c);
                        acc[i] = _mm256_fmadd_ps(a, v, acc[i]);
                    }
                }
            }
        }
        for (size_t i = 0; i < mcnt; i++) j->dst[(m0 + i) * j->n + row] = hsum256(acc[i]);
    }
}

/* reference: src/quant_matmul.rs:292-325 */
static void dot_row_avx2(const job_t *j, const float *wrow, size_t row) {
    for (size_t m0 = 0; m0 < j->m; m0 += MTILE) {
        size_t mcnt = j->m - m0 < MTILE ? j->m - m0 : MTILE;
        __m256 acc[MTILE];
        for (int i = 0; i < MTILE; i++) acc[i] = _mm256_setzero_ps();
        for (size_t c = 0; c + 8 <= j->k; c += 8) {
            __m256 wv = _mm256_loadu_ps(wrow + c);
            for (size_t i = 0; i < mcnt; i++)
                acc[i] = _mm256_fmadd_ps(_mm256_loadu_ps(j->lhs + (m0 + i) * j->k + c), wv, acc[i]);
        }
        for (size_t i = 0; i < mcnt; i++) j->dst[(m0 + i) * j->n + row] = hsum256(acc[i]);
    }
}

/* Scalar, as in the reference (src/mxfp4.rs:208-235); dst was zero-filled. */
static void row_mxfp4(const job_t *j, size_t row) {
    static const float E2M1[16] = {0.0f, 0.5f, 1.0f, 1.5f, 2.0f, 3.0f, 4.0f, 6.0f,
                                   -0.0f, -0.5f, -1.0f, -1.5f, -2.0f, -3.0f, -4.0f, -6.0f};
    const uint8_t *rb = j->blocks + row * j->bpr * 17;
    float w[32];
    for (size_t b = 0; b < j->bpr; b++) {
        const uint8_t *blk = rb + b * 17;
        int ok;
        float d = orc_e8m0(blk[0], &ok);
        if (!ok) {
            memset(w, 0, sizeof w);
        } else {
            for (int q = 0; q < 16; q++) {
                w[q] = d * E2M1[blk[1 + q] & 0xF];
                w[q + 16] = d * E2M1[blk[1 + q] >> 4];
            }
        }
        for (size_t i = 0; i < j->m; i++) {
            const float *a = j->lhs + i * j->k + b * 32;
            float acc = 0.0f;
            for (int q = 0; q < 32; q++) acc += a[q] * w[q];
            j->dst[i * j->n + row] += acc;
        }
    }
}

static void rows_worker(void *ctx, size_t rb, size_t re) {
    const job_t *j = (const job_t *)ctx;
    switch (j->type) {
    case ORC_TYPE_Q8_0:
        for (size_t r = rb; r < re; r++) row_q8_0(j, r);
        break;
    case ORC_TYPE_Q2_K:
        for (size_t r = rb; r < re; r++) row_q2_k(j, r);
        break;
    case ORC_TYPE_Q4_K:
        for (size_t r = rb; r < re; r++) row_q4_k(j, r);
        break;
    case ORC_TYPE_IQ2_XXS:
        for (size_t r = rb; r < re; r++) row_iq2_xxs(j, r);
        break;
    case ORC_TYPE_MXFP4:
        for (size_t r = rb; r < re; r++) row_mxfp4(j, r);
        break;
    case ORC_TYPE_Q6_K:
    case ORC_TYPE_Q4_0:
    case ORC_TYPE_Q4_1:
    case ORC_TYPE_Q5_0:
    case ORC_TYPE_Q5_1:
    case ORC_TYPE_Q3_K:
    case ORC_TYPE_Q5_K: {
        /* The generic path: to_float into one scratch per task, reused across its rows, then the
         * 8-lane dot (reference: src/quant_matmul.rs:229-248). */
        size_t elems, bytes;
        orc_block_geometry(j->type, &elems, &bytes);
        float *wrow = (float *)malloc(j->k * sizeof(float));
        for (size_t r = rb; r < re; r++) {
            orc_dequantize(j->type, j->blocks + r * j->bpr * bytes, j->bpr, wrow);
            dot_row_avx2(j, wrow, r);
        }
        free(wrow);
        break;
    }
    default: break;
    }
}

int orc_matmul_t_avx2(uint32_t type, size_t m, size_t k, size_t n, const float *lhs,
                      size_t lhs_len, const void *blocks, size_t nbytes, float *dst,
                      size_t dst_len, int threads) {
    size_t bpr;
    if (!orc_have_avx2()) return orc_fail("this CPU lacks AVX2/FMA/F16C");
    if (orc_validate(type, m, k, n, lhs_len, nbytes, dst_len, &bpr)) return 1;
    if (m == 0 || n == 0) return 0;
    if (threads <= 0) threads = orc_default_threads();
    pthread_once(&g_tables_once, build_tables);
    if (type == ORC_TYPE_MXFP4) memset(dst, 0, dst_len * sizeof(float));
    job_t job = {type, m, k, n, bpr, lhs, (const uint8_t *)blocks, dst};
    run_chunks(threads, n, rows_worker, &job);
    return 0;
}
