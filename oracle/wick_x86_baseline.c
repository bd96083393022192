/*
 * wick_x86_baseline.c -- what the reference executes for this path on an x86_64
 * host: the f32 fallback (no activation quantization), restated with AVX2+FMA.
 *
 * TEST/BENCH INFRASTRUCTURE ONLY: this is the "reference CPU path" timed beside
 * the GPU kernels.  It is NOT the parity oracle (different numerics: activations
 * stay f32) and the shipped library never links it.
 *
 * Follows:
 *   wick/src/backend/simd.rs:1086-1127   vec_dot_q4_0_f32_avx2
 *   wick/src/backend/simd.rs:1051-1079   vec_dot_q8_0_f32_avx2
 *   wick/src/backend/simd.rs:1198-1206   hsum_avx
 *   wick/src/backend/cpu.rs:293-306      Q4_0 GEMV row loop (serial on non-aarch64)
 *   wick/src/backend/cpu.rs:401-420      Q8_0 GEMV row loop, par_rows when m >= 256
 *   wick/src/backend/cpu.rs:222-234      par_rows: chunk = max(m / threads, 512)
 *   wick/src/model/lfm2.rs:1947-1966, 2118-2169   x86 prefill = loop of n GEMVs
 */
#include <immintrin.h>
#include <pthread.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define ORC_API __attribute__((visibility("default")))

enum { GEMV_PAR_THRESHOLD = 256 }; /* cpu.rs:310 */

static inline float hsum_avx(__m256 v) {
    __m128 hi128 = _mm256_extractf128_ps(v, 1);
    __m128 lo128 = _mm256_castps256_ps128(v);
    __m128 sum128 = _mm_add_ps(lo128, hi128);
    __m128 sum64 = _mm_add_ps(sum128, _mm_movehl_ps(sum128, sum128));
    __m128 sum32 = _mm_add_ss(sum64, _mm_shuffle_ps(sum64, sum64, 1));
    return _mm_cvtss_f32(sum32);
}

static inline float f16_bits_to_f32(uint16_t h) { return _cvtsh_ss(h); }

static inline float vec_dot_q4_0_f32_avx2(const uint8_t *blk, const float *y) {
    uint16_t hb;
    memcpy(&hb, blk, 2);
    float d = f16_bits_to_f32(hb);
    const __m256 offset = _mm256_set1_ps(8.0f);
    const __m128i mask_lo = _mm_set1_epi8(0x0F);
    __m256 sum = _mm256_setzero_ps();
    __m128i qbytes = _mm_loadu_si128((const __m128i *)(blk + 2));
    __m128i lo_bytes = _mm_and_si128(qbytes, mask_lo);
    __m128i hi_bytes = _mm_and_si128(_mm_srli_epi16(qbytes, 4), mask_lo);
    __m256 f;
    f = _mm256_sub_ps(_mm256_cvtepi32_ps(_mm256_cvtepu8_epi32(lo_bytes)), offset);
    sum = _mm256_fmadd_ps(f, _mm256_loadu_ps(y), sum);
    f = _mm256_sub_ps(_mm256_cvtepi32_ps(_mm256_cvtepu8_epi32(_mm_srli_si128(lo_bytes, 8))), offset);
    sum = _mm256_fmadd_ps(f, _mm256_loadu_ps(y + 8), sum);
    f = _mm256_sub_ps(_mm256_cvtepi32_ps(_mm256_cvtepu8_epi32(hi_bytes)), offset);
    sum = _mm256_fmadd_ps(f, _mm256_loadu_ps(y + 16), sum);
    f = _mm256_sub_ps(_mm256_cvtepi32_ps(_mm256_cvtepu8_epi32(_mm_srli_si128(hi_bytes, 8))), offset);
    sum = _mm256_fmadd_ps(f, _mm256_loadu_ps(y + 24), sum);
    return d * hsum_avx(sum);
}

static inline float vec_dot_q8_0_f32_avx2(const uint8_t *blk, const float *y) {
    uint16_t hb;
    memcpy(&hb, blk, 2);
    float d = f16_bits_to_f32(hb);
    const int8_t *q = (const int8_t *)(blk + 2);
    __m256 sum = _mm256_setzero_ps();
    for (int i = 0; i < 32; i += 8) {
        /* the reference widens the eight quants one by one into an i32 array */
        int32_t w[8];
        for (int t = 0; t < 8; t++) w[t] = q[i + t];
        __m256 qf = _mm256_cvtepi32_ps(_mm256_loadu_si256((const __m256i *)w));
        sum = _mm256_fmadd_ps(qf, _mm256_loadu_ps(y + i), sum);
    }
    return d * hsum_avx(sum);
}

static void q4_0_rows(const uint8_t *a, const float *x, float *y, int64_t r0, int64_t r1, int64_t nb) {
    for (int64_t i = r0; i < r1; i++) {
        const uint8_t *row = a + i * nb * 18;
        float sum = 0.0f;
        for (int64_t b = 0; b < nb; b++) sum += vec_dot_q4_0_f32_avx2(row + b * 18, x + b * 32);
        y[i] = sum;
    }
}

static void q8_0_rows(const uint8_t *a, const float *x, float *y, int64_t r0, int64_t r1, int64_t nb) {
    for (int64_t i = r0; i < r1; i++) {
        const uint8_t *row = a + i * nb * 34;
        float sum = 0.0f;
        for (int64_t b = 0; b < nb; b++) sum += vec_dot_q8_0_f32_avx2(row + b * 34, x + b * 32);
        y[i] = sum;
    }
}

/* cpu.rs:293-306 -- the non-aarch64 Q4_0 branch is a plain serial row loop. */
ORC_API void orc_x86_gemv_q4_0_f32(const uint8_t *a, const float *x, float *y, int64_t m, int64_t k) {
    q4_0_rows(a, x, y, 0, m, k / 32);
}

struct q8_job {
    const uint8_t *a;
    const float *x;
    float *y;
    int64_t r0, r1, nb;
};

static void *q8_worker(void *p) {
    struct q8_job *j = (struct q8_job *)p;
    q8_0_rows(j->a, j->x, j->y, j->r0, j->r1, j->nb);
    return NULL;
}

/* cpu.rs:401-420 -- Q8_0 rows go through par_rows(y, 512, ..) when m >= 256:
 * chunk = max(m / threads, 512) rows, one task per chunk (cpu.rs:222-234).
 * `threads` plays rayon's current_num_threads().  Returns the number of chunks
 * that actually ran concurrently (= cores used). */
ORC_API int orc_x86_gemv_q8_0_f32(const uint8_t *a, const float *x, float *y, int64_t m, int64_t k,
                                  int threads) {
    int64_t nb = k / 32;
    if (m < GEMV_PAR_THRESHOLD || threads <= 1) {
        q8_0_rows(a, x, y, 0, m, nb);
        return 1;
    }
    int64_t chunk = m / threads;
    if (chunk < 512) chunk = 512;
    int64_t n_chunks = (m + chunk - 1) / chunk;
    pthread_t *tid = (pthread_t *)malloc(sizeof(pthread_t) * (size_t)n_chunks);
    struct q8_job *jobs = (struct q8_job *)malloc(sizeof(struct q8_job) * (size_t)n_chunks);
    for (int64_t c = 0; c < n_chunks; c++) {
        jobs[c].a = a;
        jobs[c].x = x;
        jobs[c].y = y;
        jobs[c].r0 = c * chunk;
        jobs[c].r1 = (c + 1) * chunk < m ? (c + 1) * chunk : m;
        jobs[c].nb = nb;
        pthread_create(&tid[c], NULL, q8_worker, &jobs[c]);
    }
    for (int64_t c = 0; c < n_chunks; c++) pthread_join(tid[c], NULL);
    free(tid);
    free(jobs);
    return (int)(n_chunks < threads ? n_chunks : threads);
}

/* x86 prefill: one GEMV per token (lfm2.rs:2118-2169).  x is token-major
 * [n][k]; y is token-major [n][m]. */
ORC_API int orc_x86_prefill_f32(int ggml_type, const uint8_t *a, const float *x, float *y, int64_t m,
                                int64_t n, int64_t k, int threads) {
    int used = 1;
    for (int64_t j = 0; j < n; j++) {
        if (ggml_type == 2)
            orc_x86_gemv_q4_0_f32(a, x + j * k, y + j * m, m, k);
        else
            used = orc_x86_gemv_q8_0_f32(a, x + j * k, y + j * m, m, k, threads);
    }
    return used;
}
