/*
 * oxq_cpu_avx2.c -- TEST/BENCH INFRASTRUCTURE, NOT PRODUCT CODE.
 *
 * AVX2 intrinsics twin of the reference's SIMD fused rows, used as the CPU
 * baseline that bench.py times next to the GPU ("the reference's SIMD CPU path";
 * the reference itself is Rust and cannot be built in this image).  Same
 * instruction choices as the reference so the timing is representative:
 *   Q4_0  fused_q4_0_q8_0_row_avx2  Q/simd/avx2/q4_0.rs:190-290  (widen to i32, mullo_epi32)
 *   Q8_0  fused_q8_0_q8_0_row_avx2  Q/simd/avx2/q8_0.rs:186-256
 *   Q4_K  fused_q4k_q8_0_row_avx2   Q/simd/avx2/q4_k.rs:227-434
 *   Q6_K  fused_q6_k_q8_0_row_avx2  Q/simd/avx2/q6_k.rs:202-284  (scalar body in the reference too)
 * Q/ = /root/reference/crates/oxillama-quant/src.  Full blocks only (n_cols a
 * multiple of the block size); results are bit-identical to the oracle's
 * AVX2-tier restatement (checked in tests/test_oracle.py).
 * Threading = static row split, parallel_gemv semantics (Q/parallel.rs:70-77).
 */
#include <immintrin.h>
#include <pthread.h>
#include <stddef.h>
#include <stdint.h>

#include "oxq_oracle.h"

static inline float f16(const uint8_t *p) { return _cvtsh_ss((uint16_t)(p[0] | ((uint16_t)p[1] << 8))); }

static inline int32_t hsum_i32(__m256i v) {
    __m128i s = _mm_add_epi32(_mm256_extracti128_si256(v, 1), _mm256_castsi256_si128(v));
    s = _mm_add_epi32(s, _mm_shuffle_epi32(s, 0xB1));
    s = _mm_add_epi32(s, _mm_shuffle_epi32(s, 0x0A));
    return _mm_cvtsi128_si32(s);
}

/* sum_{i<16} w[i]*a[i] with unsigned bytes w and signed bytes a, 32-bit products */
static inline __m256i madd_u8_i8_16(__m128i w, __m128i a, __m256i acc) {
    acc = _mm256_add_epi32(acc, _mm256_mullo_epi32(_mm256_cvtepu8_epi32(w), _mm256_cvtepi8_epi32(a)));
    acc = _mm256_add_epi32(acc, _mm256_mullo_epi32(_mm256_cvtepu8_epi32(_mm_srli_si128(w, 8)),
                                                   _mm256_cvtepi8_epi32(_mm_srli_si128(a, 8))));
    return acc;
}

static float row_q4_0(const uint8_t *row, const uint8_t *acts, size_t bpr) {
    float row_sum = 0.0f;
    const __m256i eight = _mm256_set1_epi32(8);
    const __m128i mask = _mm_set1_epi8(0x0F);
    for (size_t b = 0; b < bpr; b++) {
        const uint8_t *wb = row + b * 18, *ab = acts + b * 34;
        float scale = f16(wb) * f16(ab);
        __m128i raw = _mm_loadu_si128((const __m128i *)(wb + 2));
        __m128i lo = _mm_and_si128(raw, mask), hi = _mm_and_si128(_mm_srli_epi16(raw, 4), mask);
        __m128i w0 = _mm_unpacklo_epi8(lo, hi), w1 = _mm_unpackhi_epi8(lo, hi);
        __m128i a0 = _mm_loadu_si128((const __m128i *)(ab + 2)), a1 = _mm_loadu_si128((const __m128i *)(ab + 18));
        __m256i acc = _mm256_mullo_epi32(_mm256_sub_epi32(_mm256_cvtepu8_epi32(w0), eight), _mm256_cvtepi8_epi32(a0));
        acc = _mm256_add_epi32(acc, _mm256_mullo_epi32(_mm256_sub_epi32(_mm256_cvtepu8_epi32(_mm_srli_si128(w0, 8)), eight),
                                                       _mm256_cvtepi8_epi32(_mm_srli_si128(a0, 8))));
        acc = _mm256_add_epi32(acc, _mm256_mullo_epi32(_mm256_sub_epi32(_mm256_cvtepu8_epi32(w1), eight), _mm256_cvtepi8_epi32(a1)));
        acc = _mm256_add_epi32(acc, _mm256_mullo_epi32(_mm256_sub_epi32(_mm256_cvtepu8_epi32(_mm_srli_si128(w1, 8)), eight),
                                                       _mm256_cvtepi8_epi32(_mm_srli_si128(a1, 8))));
        row_sum += scale * (float)hsum_i32(acc);
    }
    return row_sum;
}

static float row_q8_0(const uint8_t *row, const uint8_t *acts, size_t bpr) {
    float row_sum = 0.0f;
    for (size_t b = 0; b < bpr; b++) {
        const uint8_t *wb = row + b * 34, *ab = acts + b * 34;
        float scale = f16(wb) * f16(ab);
        __m128i w0 = _mm_loadu_si128((const __m128i *)(wb + 2)), w1 = _mm_loadu_si128((const __m128i *)(wb + 18));
        __m128i a0 = _mm_loadu_si128((const __m128i *)(ab + 2)), a1 = _mm_loadu_si128((const __m128i *)(ab + 18));
        __m256i acc = _mm256_mullo_epi32(_mm256_cvtepi8_epi32(w0), _mm256_cvtepi8_epi32(a0));
        acc = _mm256_add_epi32(acc, _mm256_mullo_epi32(_mm256_cvtepi8_epi32(_mm_srli_si128(w0, 8)), _mm256_cvtepi8_epi32(_mm_srli_si128(a0, 8))));
        acc = _mm256_add_epi32(acc, _mm256_mullo_epi32(_mm256_cvtepi8_epi32(w1), _mm256_cvtepi8_epi32(a1)));
        acc = _mm256_add_epi32(acc, _mm256_mullo_epi32(_mm256_cvtepi8_epi32(_mm_srli_si128(w1, 8)), _mm256_cvtepi8_epi32(_mm_srli_si128(a1, 8))));
        row_sum += scale * (float)hsum_i32(acc);
    }
    return row_sum;
}

static inline int32_t sum_i8_32(__m128i a0, __m128i a1) {
    __m256i acc = _mm256_cvtepi8_epi32(a0);
    acc = _mm256_add_epi32(acc, _mm256_cvtepi8_epi32(_mm_srli_si128(a0, 8)));
    acc = _mm256_add_epi32(acc, _mm256_cvtepi8_epi32(a1));
    acc = _mm256_add_epi32(acc, _mm256_cvtepi8_epi32(_mm_srli_si128(a1, 8)));
    return hsum_i32(acc);
}

static float row_q4_k(const uint8_t *row, const uint8_t *acts, size_t bpr) {
    float row_sum = 0.0f;
    const __m128i mask = _mm_set1_epi8(0x0F);
    for (size_t b = 0; b < bpr; b++) {
        const uint8_t *blk = row + b * 144, *s = blk + 4, *qs = blk + 16;
        float d = f16(blk), dmin = f16(blk + 2);
        uint8_t sc[8], mn[8];
        for (int j = 0; j < 4; j++) {
            sc[j] = s[j] & 0x3F;
            mn[j] = s[j + 4] & 0x3F;
            sc[j + 4] = (uint8_t)((s[j + 8] & 0x0F) | ((s[j] >> 6) << 4));
            mn[j + 4] = (uint8_t)((s[j + 8] >> 4) | ((s[j + 4] >> 6) << 4));
        }
        float block_sum = 0.0f;
        for (int g = 0; g < 4; g++) {
            const uint8_t *alo = acts + (b * 8 + 2 * (size_t)g) * 34, *ahi = alo + 34;
            float da_lo = d * (float)sc[2 * g], m_lo = dmin * (float)mn[2 * g];
            float da_hi = d * (float)sc[2 * g + 1], m_hi = dmin * (float)mn[2 * g + 1];
            __m128i r0 = _mm_loadu_si128((const __m128i *)(qs + 32 * g)), r1 = _mm_loadu_si128((const __m128i *)(qs + 32 * g + 16));
            __m128i l0 = _mm_and_si128(r0, mask), l1 = _mm_and_si128(r1, mask);
            __m128i h0 = _mm_and_si128(_mm_srli_epi16(r0, 4), mask), h1 = _mm_and_si128(_mm_srli_epi16(r1, 4), mask);
            __m128i qa0 = _mm_loadu_si128((const __m128i *)(alo + 2)), qa1 = _mm_loadu_si128((const __m128i *)(alo + 18));
            __m128i qb0 = _mm_loadu_si128((const __m128i *)(ahi + 2)), qb1 = _mm_loadu_si128((const __m128i *)(ahi + 18));
            int32_t dot_lo = hsum_i32(madd_u8_i8_16(l1, qa1, madd_u8_i8_16(l0, qa0, _mm256_setzero_si256())));
            int32_t dot_hi = hsum_i32(madd_u8_i8_16(h1, qb1, madd_u8_i8_16(h0, qb0, _mm256_setzero_si256())));
            block_sum += (da_lo * (float)dot_lo - m_lo * (float)sum_i8_32(qa0, qa1)) * f16(alo);
            block_sum += (da_hi * (float)dot_hi - m_hi * (float)sum_i8_32(qb0, qb1)) * f16(ahi);
        }
        row_sum += block_sum;
    }
    return row_sum;
}

/* The reference's "AVX2" Q6_K fused row is scalar code (Q/simd/avx2/q6_k.rs:225-281),
 * including the per-element f16 decode of the activation scale. */
static float row_q6_k(const uint8_t *row, const uint8_t *acts, size_t bpr) {
    float sum = 0.0f;
    for (size_t b = 0; b < bpr; b++) {
        const uint8_t *blk = row + b * 210, *ql = blk, *qh = blk + 128, *scales = blk + 192;
        float d = f16(blk + 208);
        for (int group = 0; group < 2; group++) {
            for (int l = 0; l < 32; l++) {
                int is = l / 16;
                uint8_t h = qh[32 * group + l];
                int32_t q[4];
                q[0] = (int32_t)(uint8_t)((ql[64 * group + l] & 0x0F) | ((h & 3) << 4)) - 32;
                q[1] = (int32_t)(uint8_t)((ql[64 * group + l + 32] & 0x0F) | (((h >> 2) & 3) << 4)) - 32;
                q[2] = (int32_t)(uint8_t)((ql[64 * group + l] >> 4) | (((h >> 4) & 3) << 4)) - 32;
                q[3] = (int32_t)(uint8_t)((ql[64 * group + l + 32] >> 4) | (((h >> 6) & 3) << 4)) - 32;
                float s[4];
                for (int j = 0; j < 4; j++) s[j] = d * (float)(int8_t)scales[8 * group + is + 2 * j];
                for (int j = 0; j < 4; j++) {
                    size_t col = (size_t)group * 128 + (size_t)l + 32 * (size_t)j;
                    const uint8_t *ab = acts + (b * 8 + col / 32) * 34;
                    float a = f16(ab) * (float)(int8_t)ab[2 + col % 32];
                    sum += s[j] * (float)q[j] * a;
                }
            }
        }
    }
    return sum;
}

typedef struct {
    uint32_t type;
    const uint8_t *w, *acts;
    float *out;
    size_t r0, r1, bpr, row_bytes;
} job_t;

static void *worker(void *p) {
    job_t *j = (job_t *)p;
    for (size_t r = j->r0; r < j->r1; r++) {
        const uint8_t *row = j->w + r * j->row_bytes;
        float v;
        switch (j->type) {
        case OXQ_REF_Q4_0: v = row_q4_0(row, j->acts, j->bpr); break;
        case OXQ_REF_Q8_0: v = row_q8_0(row, j->acts, j->bpr); break;
        case OXQ_REF_Q4_K: v = row_q4_k(row, j->acts, j->bpr); break;
        default: v = row_q6_k(row, j->acts, j->bpr); break;
        }
        j->out[r] += v; /* ACCUMULATE */
    }
    return NULL;
}

/* returns 0, or -1 for an unsupported type / partial block */
int oxq_avx2_matvec_q8_fused(uint32_t type, const uint8_t *w, const uint8_t *acts, float *out, size_t n_rows,
                             size_t n_cols, int n_threads) {
    size_t bs, bb;
    switch (type) {
    case OXQ_REF_Q4_0: bs = 32; bb = 18; break;
    case OXQ_REF_Q8_0: bs = 32; bb = 34; break;
    case OXQ_REF_Q4_K: bs = 256; bb = 144; break;
    case OXQ_REF_Q6_K: bs = 256; bb = 210; break;
    default: return -1;
    }
    if (n_cols % bs != 0) return -1;
    if (n_threads < 1) n_threads = 1;
    if (n_threads > 256) n_threads = 256;
    size_t bpr = n_cols / bs, chunk = (n_rows + (size_t)n_threads - 1) / (size_t)n_threads;
    pthread_t th[256];
    job_t jobs[256];
    int n = 0;
    for (int t = 0; t < n_threads; t++) {
        size_t r0 = (size_t)t * chunk;
        if (r0 >= n_rows) break;
        size_t r1 = r0 + chunk < n_rows ? r0 + chunk : n_rows;
        job_t j = {type, w, acts, out, r0, r1, bpr, bpr * bb};
        jobs[n] = j;
        n++;
    }
    for (int t = 1; t < n; t++) {
        if (pthread_create(&th[t], NULL, worker, &jobs[t]) != 0) {
            worker(&jobs[t]);
            th[t] = 0;
        }
    }
    if (n > 0) worker(&jobs[0]);
    for (int t = 1; t < n; t++)
        if (th[t]) pthread_join(th[t], NULL);
    return 0;
}
