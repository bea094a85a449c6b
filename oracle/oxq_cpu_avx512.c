/*
 * oxq_cpu_avx512.c -- TEST/BENCH INFRASTRUCTURE, NOT PRODUCT CODE.
 *
 * AVX-512 intrinsics twin of the reference's `gemv` on unquantized fp32 activations for Q4_K
 * (gemv_row_avx512, Q/simd/avx512/q4_k.rs:279-415; Q/ = /root/reference/crates/oxillama-quant/src), the CPU
 * figure that bench.py puts beside the GPU's fp32-activation route.  Same instruction choices so that the timing
 * is representative: per 16 weights widen the nibbles to i32, convert to fp32, w = fmsub(d * sc, q, dmin * mn),
 * acc = fmadd(w, x, acc) in one 16-lane accumulator per super-block, reduce_add per super-block, row sum over
 * super-blocks in order.  Whole super-blocks only (n_cols a multiple of 256).
 *
 * Pinned by tests/test_oracle.py against the scalar restatement (oxq_ref_gemv) within 1e-5 * max|y|: the two
 * differ in summation order (16 partial sums against one chain) and in the fused multiply-subtract.
 * Threading = static row split (Q/parallel.rs:70-77).
 */
#include <immintrin.h>
#include <pthread.h>
#include <stddef.h>
#include <stdint.h>

static inline float f16(const uint8_t *p) { return _cvtsh_ss((uint16_t)(p[0] | ((uint16_t)p[1] << 8))); }

static float gemv_row_q4_k(const uint8_t *row, const float *x, size_t bpr) {
    float row_sum = 0.0f;
    const __m128i mask = _mm_set1_epi8(0x0F);
    for (size_t b = 0; b < bpr; b++) {
        const uint8_t *blk = row + b * 144, *s = blk + 4, *qs = blk + 16;
        const float d = f16(blk), dmin = f16(blk + 2);
        uint8_t sc[8], mn[8];
        for (int j = 0; j < 4; j++) {
            sc[j] = s[j] & 0x3F;
            mn[j] = s[j + 4] & 0x3F;
            sc[j + 4] = (uint8_t)((s[j + 8] & 0x0F) | ((s[j] >> 6) << 4));
            mn[j + 4] = (uint8_t)((s[j + 8] >> 4) | ((s[j + 4] >> 6) << 4));
        }
        __m512 acc = _mm512_setzero_ps();
        const float *xb = x + b * 256;
        for (int g = 0; g < 4; g++) {
            const __m512 a_lo = _mm512_set1_ps(d * (float)sc[2 * g]), b_lo = _mm512_set1_ps(dmin * (float)mn[2 * g]);
            const __m512 a_hi = _mm512_set1_ps(d * (float)sc[2 * g + 1]), b_hi = _mm512_set1_ps(dmin * (float)mn[2 * g + 1]);
            const __m128i r0 = _mm_loadu_si128((const __m128i *)(qs + 32 * g));
            const __m128i r1 = _mm_loadu_si128((const __m128i *)(qs + 32 * g + 16));
            const __m128i nib[4] = {_mm_and_si128(r0, mask), _mm_and_si128(r1, mask),
                                    _mm_and_si128(_mm_srli_epi16(r0, 4), mask), _mm_and_si128(_mm_srli_epi16(r1, 4), mask)};
            for (int i = 0; i < 4; i++) {
                const __m512 q = _mm512_cvtepi32_ps(_mm512_cvtepu8_epi32(nib[i]));
                const __m512 w = i < 2 ? _mm512_fmsub_ps(a_lo, q, b_lo) : _mm512_fmsub_ps(a_hi, q, b_hi);
                acc = _mm512_fmadd_ps(w, _mm512_loadu_ps(xb + 64 * g + 16 * i), acc);
            }
        }
        row_sum += _mm512_reduce_add_ps(acc);
    }
    return row_sum;
}

typedef struct {
    const uint8_t *w;
    const float *x;
    float *out;
    size_t r0, r1, bpr;
} job_t;

static void *worker(void *p) {
    job_t *j = (job_t *)p;
    for (size_t r = j->r0; r < j->r1; r++) j->out[r] = gemv_row_q4_k(j->w + r * j->bpr * 144, j->x, j->bpr);
    return NULL;
}

/* out[r] = row r of W (Q4_K) . x; returns 0, or -1 for a row that ends inside a super-block */
int oxq_avx512_gemv_q4_k(const uint8_t *w, const float *x, float *out, size_t n_rows, size_t n_cols, int n_threads) {
    if (n_cols % 256 != 0) return -1;
    if (n_threads < 1) n_threads = 1;
    if (n_threads > 256) n_threads = 256;
    const size_t bpr = n_cols / 256, chunk = (n_rows + (size_t)n_threads - 1) / (size_t)n_threads;
    pthread_t th[256];
    job_t jobs[256];
    int n = 0;
    for (int t = 0; t < n_threads; t++) {
        const size_t r0 = (size_t)t * chunk;
        if (r0 >= n_rows) break;
        const job_t j = {w, x, out, r0, r0 + chunk < n_rows ? r0 + chunk : n_rows, bpr};
        jobs[n++] = j;
    }
    for (int t = 1; t < n; t++)
        if (pthread_create(&th[t], NULL, worker, &jobs[t]) != 0) {
            worker(&jobs[t]);
            th[t] = 0;
        }
    if (n > 0) worker(&jobs[0]);
    for (int t = 1; t < n; t++)
        if (th[t]) pthread_join(th[t], NULL);
    return 0;
}
