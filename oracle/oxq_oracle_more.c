/*
 * oxq_oracle_more.c -- TEST INFRASTRUCTURE, NOT PRODUCT CODE.
 *
 * Scalar C restatement of the reference's *Ref kernels (Q/reference/ = crates/oxillama-quant/
 * src/reference in /root/reference) for the formats beyond the first five: Q4_1, Q5_0, Q5_1,
 * Q8_1, IQ4_NL, Q2_K, Q3_K, Q5_K.  dequant_block, gemv and matvec_q8_fused follow the cited
 * lines operation for operation (fp32, no contraction); Q4_1 and IQ4_NL have no
 * matvec_q8_fused of their own and take the trait default (Q/traits.rs:137-170).
 * Tail columns: every caller passes n_cols that is a block multiple except the gemv / fused
 * row functions, which skip columns >= n_cols as the reference does.
 *
 * Pinning (tests/test_oracle_more.py): the reference's hand-built block tests of each file,
 * independent numpy decoders written from the format definitions, gemv == sum dequant * x in
 * float64, fused == gemv on dequantized activations, brute-force integer sums.
 */
#include <string.h>

#include "oxq_oracle.h"
#include "oxq_oracle_more.h"

enum { T_Q4_1 = 3, T_Q5_0 = 6, T_Q5_1 = 7, T_Q8_1 = 9, T_Q2_K = 10, T_Q3_K = 11, T_Q5_K = 13, T_IQ4_NL = 20 };

static float h(const uint8_t *p) { return oxq_ref_f16_to_f32((uint16_t)(p[0] | ((uint16_t)p[1] << 8))); }
static uint32_t u32le(const uint8_t *p) {
    return (uint32_t)p[0] | ((uint32_t)p[1] << 8) | ((uint32_t)p[2] << 16) | ((uint32_t)p[3] << 24);
}

/* KVALUES_IQ4NL, Q/reference/iq_shared.rs:16-18 */
static const int8_t KV[16] = {-127, -104, -83, -65, -49, -35, -22, -10, 1, 13, 25, 38, 53, 69, 89, 113};

int oxq_more_known(uint32_t t) { return oxq_more_block_size(t) != 0; }

size_t oxq_more_block_size(uint32_t t) {
    switch (t) {
    case T_Q4_1: case T_Q5_0: case T_Q5_1: case T_Q8_1: case T_IQ4_NL: return 32;
    case T_Q2_K: case T_Q3_K: case T_Q5_K: return 256;
    default: return 0;
    }
}

size_t oxq_more_block_bytes(uint32_t t) {
    switch (t) {
    case T_Q4_1: return 20;  /* Q/reference/q4_1.rs:17 */
    case T_Q5_0: return 22;  /* q5_0.rs:18 */
    case T_Q5_1: return 24;  /* q5_1.rs:19 */
    case T_Q8_1: return 36;  /* q8_1.rs:17 */
    case T_IQ4_NL: return 18; /* iq4_nl.rs:22 */
    case T_Q2_K: return 84;  /* q2_k.rs:21 */
    case T_Q3_K: return 110; /* q3_k.rs:21 */
    case T_Q5_K: return 176; /* q5_k.rs:20 */
    default: return 0;
    }
}

size_t oxq_more_groups_per_block(uint32_t t) {
    switch (t) {
    case T_Q2_K: case T_Q3_K: return 16;
    case T_Q5_K: return 8;
    default: return 1;
    }
}

/* 6-bit scales / mins of Q5_K: decode_scales_mins, q5_k.rs:27-49 (same packing as Q4_K) */
static void q5k_scales_mins(const uint8_t *s, uint8_t sc[8], uint8_t mn[8]) {
    for (int j = 0; j < 4; j++) {
        sc[j] = s[j] & 0x3F;
        mn[j] = s[j + 4] & 0x3F;
    }
    for (int j = 4; j < 8; j++) {
        sc[j] = (uint8_t)((s[j + 4] & 0x0F) | (((s[j - 4] >> 6) & 0x03) << 4));
        mn[j] = (uint8_t)(((s[j + 4] >> 4) & 0x0F) | (((s[j] >> 6) & 0x03) << 4));
    }
}

/* decode_scales, q3_k.rs:30-59: 16 six-bit values minus 32, as floats */
static void q3k_scales(const uint8_t *s, float out[16]) {
    uint32_t sc[16];
    for (int j = 0; j < 4; j++) sc[j] = s[j] & 0x3F;
    for (int j = 0; j < 4; j++) sc[4 + j] = s[4 + j] & 0x3F;
    for (int j = 0; j < 4; j++) sc[8 + j] = (uint32_t)(s[8 + j] & 0x0F) | ((uint32_t)((s[j] >> 6) & 0x03) << 4);
    for (int j = 0; j < 4; j++) sc[12 + j] = (uint32_t)((s[8 + j] >> 4) & 0x0F) | ((uint32_t)((s[4 + j] >> 6) & 0x03) << 4);
    for (int i = 0; i < 16; i++) out[i] = (float)((int32_t)sc[i] - 32);
}

/* ---- integer weights of one block, in column order (the integer view every test shares) ---- */
/* Q4_1: nibble; Q5_0: q5 - 16; Q5_1: q5; Q8_1: int8; IQ4_NL: codebook value; Q2_K: q2; Q3_K: q_lo - (hmask ? 0 : 4);
 * Q5_K: q5. */
static void int_weights(uint32_t t, const uint8_t *b, int32_t *q) {
    switch (t) {
    case T_Q4_1:
        for (int i = 0; i < 16; i++) { q[2 * i] = b[4 + i] & 0x0F; q[2 * i + 1] = b[4 + i] >> 4; }
        break;
    case T_Q5_0: {
        uint32_t qh = u32le(b + 2);
        for (int i = 0; i < 16; i++) {
            q[i] = (int32_t)((b[6 + i] & 0x0F) | (((qh >> i) & 1) << 4)) - 16;
            q[i + 16] = (int32_t)((b[6 + i] >> 4) | (((qh >> (i + 16)) & 1) << 4)) - 16;
        }
        break;
    }
    case T_Q5_1: {
        uint32_t qh = u32le(b + 4);
        for (int i = 0; i < 16; i++) {
            q[i] = (int32_t)((b[8 + i] & 0x0F) | (((qh >> i) & 1) << 4));
            q[i + 16] = (int32_t)((b[8 + i] >> 4) | (((qh >> (i + 16)) & 1) << 4));
        }
        break;
    }
    case T_Q8_1:
        for (int i = 0; i < 32; i++) q[i] = (int8_t)b[4 + i];
        break;
    case T_IQ4_NL:
        for (int i = 0; i < 16; i++) { q[2 * i] = KV[b[2 + i] & 0x0F]; q[2 * i + 1] = KV[b[2 + i] >> 4]; }
        break;
    case T_Q2_K: {
        const uint8_t *qs = b + 16;
        int o = 0;
        for (int n = 0; n < 2; n++)
            for (int shift = 0; shift < 8; shift += 2)
                for (int half = 0; half < 2; half++)
                    for (int l = 0; l < 16; l++) q[o++] = (qs[32 * n + 16 * half + l] >> shift) & 3;
        break;
    }
    case T_Q3_K: {
        const uint8_t *hm = b, *qs = b + 32;
        int o = 0;
        uint8_t m = 1;
        for (int g = 0; g < 2; g++)
            for (int shift = 0; shift < 8; shift += 2) {
                for (int n = 0; n < 2; n++)
                    for (int l = 0; l < 16; l++) {
                        int32_t lo = (qs[32 * g + 16 * n + l] >> shift) & 3;
                        q[o++] = lo - ((hm[16 * n + l] & m) ? 0 : 4);
                    }
                m = (uint8_t)(m << 1);
            }
        break;
    }
    case T_Q5_K: {
        const uint8_t *qh = b + 16, *qs = b + 48;
        for (int g = 0; g < 4; g++)
            for (int l = 0; l < 32; l++) {
                q[64 * g + l] = (qs[32 * g + l] & 0x0F) | (((qh[l] >> g) & 1) << 4);
                q[64 * g + 32 + l] = (qs[32 * g + l] >> 4) | (((qh[l] >> (g + 4)) & 1) << 4);
            }
        break;
    }
    default: break;
    }
}

/* ---- dequant_block ---- */
void oxq_more_dequant(uint32_t t, const uint8_t *b, float *out) {
    int32_t q[256];
    int_weights(t, b, q);
    switch (t) {
    case T_Q4_1: { /* q4_1.rs:37-46: d * nibble + m */
        float d = h(b), m = h(b + 2);
        for (int i = 0; i < 32; i++) out[i] = d * (float)q[i] + m;
        break;
    }
    case T_Q5_0: { /* q5_0.rs:39-55: d * (q5 - 16) */
        float d = h(b);
        for (int i = 0; i < 32; i++) out[i] = d * (float)q[i];
        break;
    }
    case T_Q5_1: { /* q5_1.rs:38-56: d * q5 + m */
        float d = h(b), m = h(b + 2);
        for (int i = 0; i < 32; i++) out[i] = d * (float)q[i] + m;
        break;
    }
    case T_Q8_1: { /* q8_1.rs:36-42 */
        float d = h(b);
        for (int i = 0; i < 32; i++) out[i] = d * (float)q[i];
        break;
    }
    case T_IQ4_NL: { /* iq4_nl.rs:43-51: d * kvalues[idx] */
        float d = h(b);
        for (int i = 0; i < 32; i++) out[i] = d * (float)q[i];
        break;
    }
    case T_Q2_K: { /* q2_k.rs:41-80: dl * q - ml, dl = d * (sc & 15), ml = dmin * (sc >> 4) */
        float d = h(b + 80), dmin = h(b + 82);
        for (int is = 0; is < 16; is++) {
            float dl = d * (float)(b[is] & 0x0F), ml = dmin * (float)(b[is] >> 4);
            for (int l = 0; l < 16; l++) out[16 * is + l] = dl * (float)q[16 * is + l] - ml;
        }
        break;
    }
    case T_Q3_K: { /* q3_k.rs:76-120: (d * sc) * (q_lo - sub) */
        float sc[16], d = h(b + 108);
        q3k_scales(b + 96, sc);
        for (int is = 0; is < 16; is++) {
            float dl = d * sc[is];
            for (int l = 0; l < 16; l++) out[16 * is + l] = dl * (float)q[16 * is + l];
        }
        break;
    }
    case T_Q5_K: { /* q5_k.rs:66-102: d1 * q - m1 */
        uint8_t sc[8], mn[8];
        float d = h(b), dmin = h(b + 2);
        q5k_scales_mins(b + 4, sc, mn);
        for (int s = 0; s < 8; s++) {
            float d1 = d * (float)sc[s], m1 = dmin * (float)mn[s];
            for (int l = 0; l < 32; l++) out[32 * s + l] = d1 * (float)q[32 * s + l] - m1;
        }
        break;
    }
    default: break;
    }
}

/* ---- gemv rows (fp32 activations), each format's own operation order ---- */
float oxq_more_gemv_row(uint32_t t, const uint8_t *row, size_t bpr, size_t n_cols, const float *x) {
    const size_t bs = oxq_more_block_size(t), bb = oxq_more_block_bytes(t);
    float sum = 0.0f;
    int32_t q[256];
    for (size_t blk = 0; blk < bpr; blk++) {
        const uint8_t *b = row + blk * bb;
        const float *inp = x + blk * bs;
        const size_t rem = n_cols - blk * bs < bs ? n_cols - blk * bs : bs;
        int_weights(t, b, q);
        switch (t) {
        case T_Q4_1: { /* q4_1.rs gemv: sum += d * lo * inp[j]; input_sum; sum += m * input_sum */
            float d = h(b), m = h(b + 2), input_sum = 0.0f;
            for (size_t j = 0; j < 32; j++)
                if (j < rem) { sum += d * (float)q[j] * inp[j]; input_sum += inp[j]; }
            sum += m * input_sum;
            break;
        }
        case T_Q5_0: { /* q5_0.rs gemv: pairs (i, i+16) in turn */
            float d = h(b);
            for (size_t i = 0; i < 16; i++) {
                sum += d * (float)q[i] * inp[i];
                sum += d * (float)q[i + 16] * inp[i + 16];
            }
            break;
        }
        case T_Q5_1: { /* q5_1.rs gemv */
            float d = h(b), m = h(b + 2), input_sum = 0.0f;
            for (size_t i = 0; i < 16; i++) {
                if (i < rem) { sum += d * (float)q[i] * inp[i]; input_sum += inp[i]; }
                if (i + 16 < rem) { sum += d * (float)q[i + 16] * inp[i + 16]; input_sum += inp[i + 16]; }
            }
            sum += m * input_sum;
            break;
        }
        case T_Q8_1: { /* q8_1.rs gemv: block_sum of q * x, then d * block_sum */
            float d = h(b), bsum = 0.0f;
            for (size_t i = 0; i < 32; i++) bsum += (float)q[i] * inp[i];
            sum += d * bsum;
            break;
        }
        case T_IQ4_NL: { /* iq4_nl.rs gemv: kv as f32 * d * x */
            float d = h(b);
            for (size_t i = 0; i < 32; i++)
                if (i < rem) sum += (float)q[i] * d * inp[i];
            break;
        }
        case T_Q2_K: { /* q2_k.rs gemv: (dl * q - ml) * x */
            float d = h(b + 80), dmin = h(b + 82);
            for (size_t is = 0; is < 16; is++) {
                float dl = d * (float)(b[is] & 0x0F), ml = dmin * (float)(b[is] >> 4);
                for (size_t l = 0; l < 16; l++)
                    if (16 * is + l < rem) sum += (dl * (float)q[16 * is + l] - ml) * inp[16 * is + l];
            }
            break;
        }
        case T_Q3_K: { /* q3_k.rs gemv: dl * q3 * x */
            float sc[16], d = h(b + 108);
            q3k_scales(b + 96, sc);
            for (size_t is = 0; is < 16; is++) {
                float dl = d * sc[is];
                for (size_t l = 0; l < 16; l++)
                    if (16 * is + l < rem) sum += dl * (float)q[16 * is + l] * inp[16 * is + l];
            }
            break;
        }
        case T_Q5_K: { /* q5_k.rs:166-199: (d1 * q - m1) * x */
            uint8_t sc[8], mn[8];
            float d = h(b), dmin = h(b + 2);
            q5k_scales_mins(b + 4, sc, mn);
            for (size_t s = 0; s < 8; s++) {
                float d1 = d * (float)sc[s], m1 = dmin * (float)mn[s];
                for (size_t l = 0; l < 32; l++)
                    if (32 * s + l < rem) sum += (d1 * (float)q[32 * s + l] - m1) * inp[32 * s + l];
            }
            break;
        }
        default: break;
        }
    }
    return sum;
}

/* ---- matvec_q8_fused rows ---- */
float oxq_more_fused_row(uint32_t t, const uint8_t *row, size_t bpr, size_t n_cols, const uint8_t *acts) {
    const size_t bs = oxq_more_block_size(t), bb = oxq_more_block_bytes(t);
    float sum = 0.0f;
    int32_t q[256];
    for (size_t blk = 0; blk < bpr; blk++) {
        const uint8_t *b = row + blk * bb;
        const size_t rem = n_cols - blk * bs < bs ? n_cols - blk * bs : bs;
        int_weights(t, b, q);
        switch (t) {
        case T_Q4_1:
        case T_IQ4_NL: { /* trait default, Q/traits.rs:137-170 */
            float w[32], a[32];
            oxq_more_dequant(t, b, w);
            const uint8_t *ab = acts + blk * 34;
            float d_a = h(ab);
            for (size_t i = 0; i < rem; i++) a[i] = (float)(int8_t)ab[2 + i] * d_a;
            for (size_t i = 0; i < rem; i++) sum += w[i] * a[i];
            break;
        }
        case T_Q5_0: { /* q5_0.rs:189-230: dot += d_w * q * (q_a * d_a), pairs (i, i+16); sum += dot */
            const uint8_t *ab = acts + blk * 34;
            float d_w = h(b), d_a = h(ab), dot = 0.0f;
            for (size_t i = 0; i < 16; i++) {
                if (i >= rem && i + 16 >= rem) break;
                if (i < rem) { float a0 = (float)(int8_t)ab[2 + i] * d_a; dot += d_w * (float)q[i] * a0; }
                if (i + 16 < rem) { float a1 = (float)(int8_t)ab[2 + i + 16] * d_a; dot += d_w * (float)q[i + 16] * a1; }
            }
            sum += dot;
            break;
        }
        case T_Q5_1: { /* q5_1.rs:200-245: dot and inp_sum; sum += dot + m_w * inp_sum */
            const uint8_t *ab = acts + blk * 34;
            float d_w = h(b), m_w = h(b + 2), d_a = h(ab), dot = 0.0f, inp_sum = 0.0f;
            for (size_t i = 0; i < 16; i++) {
                if (i < rem) { float a0 = (float)(int8_t)ab[2 + i] * d_a; dot += d_w * (float)q[i] * a0; inp_sum += a0; }
                if (i + 16 < rem) {
                    float a1 = (float)(int8_t)ab[2 + i + 16] * d_a;
                    dot += d_w * (float)q[i + 16] * a1;
                    inp_sum += a1;
                }
            }
            sum += dot + m_w * inp_sum;
            break;
        }
        case T_Q8_1: { /* q8_1.rs:170-200: dot += w * (q_a * d_a); sum += d_w * dot */
            const uint8_t *ab = acts + blk * 34;
            float d_w = h(b), d_a = h(ab), dot = 0.0f;
            for (size_t i = 0; i < rem; i++) dot += (float)q[i] * ((float)(int8_t)ab[2 + i] * d_a);
            sum += d_w * dot;
            break;
        }
        case T_Q2_K: { /* q2_k.rs:224-292: per 16 weights (dl * dot - ml * sum_a) * d_a */
            float d = h(b + 80), dmin = h(b + 82);
            for (size_t is = 0; is < 16; is++) {
                float dl = d * (float)(b[is] & 0x0F), ml = dmin * (float)(b[is] >> 4);
                const uint8_t *ab = acts + (blk * 8 + is / 2) * 34;
                float d_a = h(ab), dot = 0.0f, sum_a = 0.0f;
                for (size_t l = 0; l < 16; l++)
                    if (16 * is + l < rem) {
                        float q_a = (float)(int8_t)ab[2 + 16 * (is & 1) + l];
                        dot += (float)q[16 * is + l] * q_a;
                        sum_a += q_a;
                    }
                sum += (dl * dot - ml * sum_a) * d_a;
            }
            break;
        }
        case T_Q3_K: { /* q3_k.rs:258-322: per 16 weights dl * dot * d_a */
            float sc[16], d = h(b + 108);
            q3k_scales(b + 96, sc);
            for (size_t is = 0; is < 16; is++) {
                float dl = d * sc[is];
                const uint8_t *ab = acts + (blk * 8 + is / 2) * 34;
                float d_a = h(ab), dot = 0.0f;
                for (size_t l = 0; l < 16; l++)
                    if (16 * is + l < rem) dot += (float)q[16 * is + l] * (float)(int8_t)ab[2 + 16 * (is & 1) + l];
                sum += dl * dot * d_a;
            }
            break;
        }
        case T_Q5_K: { /* q5_k.rs:270-345: per 32 weights (da * dot - m * sum_a) * d_a */
            uint8_t sc[8], mn[8];
            float d = h(b), dmin = h(b + 2);
            q5k_scales_mins(b + 4, sc, mn);
            for (size_t s = 0; s < 8; s++) {
                const uint8_t *ab = acts + (blk * 8 + s) * 34;
                float d_a = h(ab), da = d * (float)sc[s], m = dmin * (float)mn[s], dot = 0.0f, sum_a = 0.0f;
                for (size_t l = 0; l < 32; l++)
                    if (32 * s + l < rem) {
                        float q_a = (float)(int8_t)ab[2 + l];
                        dot += (float)q[32 * s + l] * q_a;
                        sum_a += q_a;
                    }
                sum += (da * dot - m * sum_a) * d_a;
            }
            break;
        }
        default: break;
        }
    }
    return sum;
}

/* ---- exact integer sums per group: sum of int_weights * q_a over 32 (16 for Q2_K, Q3_K) columns ---- */
void oxq_more_block_sums_row(uint32_t t, const uint8_t *row, size_t bpr, const uint8_t *acts, int32_t *sums) {
    const size_t bs = oxq_more_block_size(t), bb = oxq_more_block_bytes(t);
    const size_t gpb = oxq_more_groups_per_block(t), gcols = bs / gpb;
    int32_t q[256];
    for (size_t blk = 0; blk < bpr; blk++) {
        int_weights(t, row + blk * bb, q);
        for (size_t g = 0; g < gpb; g++) {
            int32_t s = 0;
            for (size_t l = 0; l < gcols; l++) {
                size_t col = blk * bs + g * gcols + l;
                s += q[g * gcols + l] * (int32_t)(int8_t)acts[(col / 32) * 34 + 2 + col % 32];
            }
            sums[blk * gpb + g] = s;
        }
    }
}

/* Integer-dot form: one fp32 term per group from the exact sums (what a kernel that multiplies
 * in the integer domain computes), groups left to right. */
float oxq_more_intdot_row(uint32_t t, const uint8_t *row, size_t bpr, const uint8_t *acts, int32_t *scratch) {
    const size_t bs = oxq_more_block_size(t), bb = oxq_more_block_bytes(t);
    const size_t gpb = oxq_more_groups_per_block(t), gcols = bs / gpb;
    oxq_more_block_sums_row(t, row, bpr, acts, scratch);
    float sum = 0.0f;
    for (size_t blk = 0; blk < bpr; blk++) {
        const uint8_t *b = row + blk * bb;
        float q3sc[16];
        uint8_t sc[8], mn[8];
        if (t == T_Q3_K) q3k_scales(b + 96, q3sc);
        if (t == T_Q5_K) q5k_scales_mins(b + 4, sc, mn);
        for (size_t g = 0; g < gpb; g++) {
            size_t col0 = blk * bs + g * gcols;
            const uint8_t *ab = acts + (col0 / 32) * 34;
            float d_a = h(ab), isum = (float)scratch[blk * gpb + g];
            int32_t asum = 0;
            for (size_t l = 0; l < gcols; l++) asum += (int8_t)ab[2 + col0 % 32 + l];
            switch (t) {
            case T_Q4_1:
            case T_Q5_1: sum += (h(b) * isum + h(b + 2) * (float)asum) * d_a; break;
            case T_Q5_0:
            case T_Q8_1:
            case T_IQ4_NL: sum += h(b) * isum * d_a; break;
            case T_Q2_K:
                sum += (h(b + 80) * (float)(b[g] & 0x0F) * isum - h(b + 82) * (float)(b[g] >> 4) * (float)asum) * d_a;
                break;
            case T_Q3_K: sum += h(b + 108) * q3sc[g] * isum * d_a; break;
            case T_Q5_K: sum += (h(b) * (float)sc[g] * isum - h(b + 2) * (float)mn[g] * (float)asum) * d_a; break;
            default: break;
            }
        }
    }
    return sum;
}
