/*
 * fnn_cpu_baseline.c -- a CPU implementation of fastnn's packed MatMul tuned the way the reference's own
 * benchmark rows were produced: AVX2 unpack of a weight row to f32 + FMA dot products, rows of the weight
 * spread over threads.  Test infrastructure (bench.py's cpu_baseline leg and its test only); never linked
 * into the product.
 *
 * What it follows in the reference (paths relative to the fastnn tree):
 *   - gemm_batch_packed_simd, src/backend/cpu/microkernels/gemm.rs:1982-2088: each weight row is unpacked
 *     once and dotted with every activation row (fma_f32_slice), then the affine epilogue
 *     out = dot*scale + zero*sum(a) (apply_affine_dot, src/backend/cpu/microkernels/mod.rs:283-295);
 *   - the unpack kernels CHANGELOG.md:620-622 names: int8 -> f32 widening with _mm256_cvtepi8_epi32, 4-bit
 *     lanes by shift / mask / sign extension;
 *   - threading: the published GEMV rows (CHANGELOG.md:628-635, "8 threads") spread weight rows over the
 *     pool; today's gemm_batch_packed_simd only goes parallel over activation rows when there are at least
 *     `physical cores` of them, i.e. runs M = 1 on one thread.  Both are available here: `threads` = 1
 *     reproduces today's M = 1 behaviour, `threads` > 1 the published set-up.
 *
 * The summation order differs from the oracle's restatement (four 8-lane accumulators), so results agree with
 * it to f32 rounding only (checked in tests/test_oracle_matmul.py at 1e-5 of max|out|).
 * Build: gcc -O3 -mavx2 -mfma -pthread (see Makefile); returns -2 at run time on a CPU without AVX2/FMA.
 */
#include <immintrin.h>
#include <math.h>
#include <pthread.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

enum { DT_I8 = 0, DT_I4 = 1 };

typedef struct {
    int dt;
    const uint32_t *words;
    int64_t n, k, kp;
    const float *scales, *zeros, *a, *bias, *asum;
    int64_t m;
    int act;
    float *out;
    int64_t row0, row1;
    float *buf; /* k floats (padded to 8) */
} job_t;

static inline float hsum8(__m256 v)
{
    __m128 lo = _mm256_castps256_ps128(v), hi = _mm256_extractf128_ps(v, 1);
    lo = _mm_add_ps(lo, hi);
    lo = _mm_hadd_ps(lo, lo);
    lo = _mm_hadd_ps(lo, lo);
    return _mm_cvtss_f32(lo);
}

static void unpack_row_i8(const uint32_t *w, int64_t kp, float *buf)
{
    const int8_t *b = (const int8_t *)w;
    int64_t nb = kp * 4, i = 0;
    for (; i + 8 <= nb; i += 8) {
        __m128i v = _mm_loadl_epi64((const __m128i *)(b + i));
        _mm256_storeu_ps(buf + i, _mm256_cvtepi32_ps(_mm256_cvtepi8_epi32(v)));
    }
    for (; i < nb; i++) buf[i] = (float)b[i];
}

static void unpack_row_i4(const uint32_t *w, int64_t kp, float *buf)
{
    const __m256i sh = _mm256_setr_epi32(0, 4, 8, 12, 16, 20, 24, 28);
    const __m256i m4 = _mm256_set1_epi32(15), eight = _mm256_set1_epi32(8);
    for (int64_t p = 0; p < kp; p++) {
        __m256i v = _mm256_and_si256(_mm256_srlv_epi32(_mm256_set1_epi32((int)w[p]), sh), m4);
        v = _mm256_sub_epi32(_mm256_xor_si256(v, eight), eight); /* sign-extend the nibble */
        _mm256_storeu_ps(buf + p * 8, _mm256_cvtepi32_ps(v));
    }
}

static float dot_avx2(const float *x, const float *y, int64_t k)
{
    __m256 a0 = _mm256_setzero_ps(), a1 = a0, a2 = a0, a3 = a0;
    int64_t i = 0;
    for (; i + 32 <= k; i += 32) {
        a0 = _mm256_fmadd_ps(_mm256_loadu_ps(x + i), _mm256_loadu_ps(y + i), a0);
        a1 = _mm256_fmadd_ps(_mm256_loadu_ps(x + i + 8), _mm256_loadu_ps(y + i + 8), a1);
        a2 = _mm256_fmadd_ps(_mm256_loadu_ps(x + i + 16), _mm256_loadu_ps(y + i + 16), a2);
        a3 = _mm256_fmadd_ps(_mm256_loadu_ps(x + i + 24), _mm256_loadu_ps(y + i + 24), a3);
    }
    for (; i + 8 <= k; i += 8) a0 = _mm256_fmadd_ps(_mm256_loadu_ps(x + i), _mm256_loadu_ps(y + i), a0);
    float s = hsum8(_mm256_add_ps(_mm256_add_ps(a0, a1), _mm256_add_ps(a2, a3)));
    for (; i < k; i++) s += x[i] * y[i];
    return s;
}

static float activate(float v, int act)
{
    switch (act) {
    case 1: return v > 0.0f ? v : 0.0f;
    case 2: { /* tanh form of GELU, src/backend/cpu/microkernels/conv_gemm.rs:121-143 */
        float x3 = v * v * v;
        return 0.5f * v * (1.0f + tanhf(0.7978846f * (v + 0.044715f * x3)));
    }
    case 3: return v / (1.0f + expf(-v));
    default: return v;
    }
}

static void *worker(void *arg)
{
    job_t *j = (job_t *)arg;
    for (int64_t r = j->row0; r < j->row1; r++) {
        if (j->dt == DT_I8) unpack_row_i8(j->words + r * j->kp, j->kp, j->buf);
        else unpack_row_i4(j->words + r * j->kp, j->kp, j->buf);
        const float sc = j->scales[r], zr = j->zeros ? j->zeros[r] : 0.0f;
        for (int64_t b = 0; b < j->m; b++) {
            float v = dot_avx2(j->buf, j->a + b * j->k, j->k) * sc + zr * j->asum[b];
            if (j->bias) v += j->bias[r];
            j->out[b * j->n + r] = activate(v, j->act);
        }
    }
    return NULL;
}

/* out[m,n] = act((sum_k a[m,k]*q[n,k])*scale[n] + zero[n]*sum_k a[m,k] + bias[n]); dt: 0 = I8x4, 1 = I4x8.
 * Returns 0, -1 for another dtype or bad arguments, -2 without AVX2/FMA, -3 when out of memory. */
int fnn_cpu_qgemm(int dt, const uint32_t *words, int64_t n, int64_t k, const float *scales, const float *zeros,
                  const float *a, int64_t m, const float *bias, int act, float *out, int threads)
{
    if ((dt != DT_I8 && dt != DT_I4) || !words || !scales || !a || !out || n <= 0 || k <= 0 || m <= 0) return -1;
    if (!__builtin_cpu_supports("avx2") || !__builtin_cpu_supports("fma")) return -2;
    if (threads < 1) threads = 1;
    if (threads > 256) threads = 256;
    if (threads > n) threads = (int)n;
    const int items = dt == DT_I8 ? 4 : 8;
    const int64_t kp = (k + items - 1) / items;
    float *asum = (float *)malloc(sizeof(float) * (size_t)m);
    job_t *jobs = (job_t *)calloc((size_t)threads, sizeof(job_t));
    pthread_t *tids = (pthread_t *)calloc((size_t)threads, sizeof(pthread_t));
    if (!asum || !jobs || !tids) { free(asum); free(jobs); free(tids); return -3; }
    for (int64_t b = 0; b < m; b++) { /* affine_sum_term: sum of the activation row */
        float s = 0.0f;
        for (int64_t i = 0; i < k; i++) s += a[b * k + i];
        asum[b] = s;
    }
    int rc = 0, started = 0;
    for (int t = 0; t < threads; t++) {
        job_t *j = &jobs[t];
        j->dt = dt; j->words = words; j->n = n; j->k = k; j->kp = kp; j->scales = scales; j->zeros = zeros;
        j->a = a; j->bias = bias; j->asum = asum; j->m = m; j->act = act; j->out = out;
        j->row0 = n * t / threads; j->row1 = n * (t + 1) / threads;
        j->buf = (float *)aligned_alloc(64, (size_t)((kp * items + 15) / 16 * 16) * sizeof(float));
        if (!j->buf) { rc = -3; break; }
        if (threads == 1) { worker(j); continue; }
        if (pthread_create(&tids[t], NULL, worker, j) != 0) { rc = -3; break; }
        started++;
    }
    for (int t = 0; t < started; t++) pthread_join(tids[t], NULL);
    for (int t = 0; t < threads; t++) free(jobs[t].buf);
    free(asum); free(jobs); free(tids);
    return rc;
}
