/*
 * oxq_oracle.c -- TEST INFRASTRUCTURE, NOT PRODUCT CODE (see oxq_oracle.h).
 *
 * Scalar restatement of the reference CPU kernels, in the reference's operation
 * order.  Q/ = /root/reference/crates/oxillama-quant/src.
 */
#include "oxq_oracle.h"
#include "oxq_oracle_more.h"

#include <math.h>
#include <stdlib.h>
#include <string.h>

#define Q8_0_BLOCK_BYTES 34 /* Q/traits.rs:12 */

static oxq_ref_status ok(void) {
    oxq_ref_status s = {OXQ_REF_OK, 0, 0};
    return s;
}
static oxq_ref_status err(int code, size_t a, size_t b) {
    oxq_ref_status s = {code, a, b};
    return s;
}

/* crates/oxillama-gguf/src/types.rs:199-216 */
size_t oxq_ref_block_size(uint32_t type) {
    switch (type) {
    case OXQ_REF_Q4_0:
    case OXQ_REF_Q8_0:
        return 32;
    case OXQ_REF_Q4_K:
    case OXQ_REF_Q6_K:
    case OXQ_REF_IQ4_XS:
        return 256;
    default:
        return oxq_more_block_size(type);
    }
}

/* crates/oxillama-gguf/src/types.rs:219-262 */
size_t oxq_ref_block_bytes(uint32_t type) {
    switch (type) {
    case OXQ_REF_Q4_0:
        return 18;
    case OXQ_REF_Q8_0:
        return 34;
    case OXQ_REF_Q4_K:
        return 144;
    case OXQ_REF_Q6_K:
        return 210;
    case OXQ_REF_IQ4_XS:
        return 136;
    default:
        return oxq_more_block_bytes(type);
    }
}

/* ---- half::f16 (crate `half` 2.x; IEEE binary16, round-to-nearest-even) ---- */

float oxq_ref_f16_to_f32(uint16_t h) {
    uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1Fu;
    uint32_t man = h & 0x3FFu;
    uint32_t bits;
    if (exp == 0) {
        if (man == 0) {
            bits = sign;
        } else {
            /* subnormal: value = man * 2^-24, normalise */
            int e = -1;
            do {
                e++;
                man <<= 1;
            } while ((man & 0x400u) == 0);
            bits = sign | ((uint32_t)(127 - 15 - e) << 23) | ((man & 0x3FFu) << 13);
        }
    } else if (exp == 31) {
        bits = sign | 0x7F800000u | (man << 13);
    } else {
        bits = sign | ((exp + 127 - 15) << 23) | (man << 13);
    }
    float f;
    memcpy(&f, &bits, 4);
    return f;
}

uint16_t oxq_ref_f32_to_f16(float v) {
    uint32_t x;
    memcpy(&x, &v, 4);
    uint32_t sign = (x >> 16) & 0x8000u;
    uint32_t exp = (x >> 23) & 0xFFu;
    uint32_t man = x & 0x7FFFFFu;
    if (exp == 0xFF) {
        /* Inf / NaN: keep NaN-ness (set the quiet bit), keep top payload bits */
        uint32_t nan_bit = man ? 0x0200u : 0;
        return (uint16_t)(sign | 0x7C00u | nan_bit | (man >> 13));
    }
    int32_t e = (int32_t)exp - 127 + 15;
    if (e >= 31) {
        return (uint16_t)(sign | 0x7C00u); /* overflow -> inf */
    }
    if (e <= 0) {
        if (e < -10) {
            return (uint16_t)sign; /* too small even for a subnormal: +-0 */
        }
        /* subnormal result: shift the 24-bit significand, round to nearest even */
        man |= 0x800000u;
        uint32_t shift = (uint32_t)(14 - e); /* 14..24 */
        uint32_t half_man = man >> shift;
        uint32_t rem = man & ((1u << shift) - 1u);
        uint32_t halfway = 1u << (shift - 1);
        if (rem > halfway || (rem == halfway && (half_man & 1u))) {
            half_man++;
        }
        return (uint16_t)(sign | half_man);
    }
    uint32_t half = ((uint32_t)e << 10) | (man >> 13);
    uint32_t rem = man & 0x1FFFu;
    if (rem > 0x1000u || (rem == 0x1000u && (half & 1u))) {
        half++; /* may carry into the exponent, up to inf: correct */
    }
    return (uint16_t)(sign | half);
}

static float rd_f16(const uint8_t *p) {
    /* u16::from_le_bytes([p[0], p[1]]) then f16::to_f32, Q/reference/q4_k.rs:351-353 */
    return oxq_ref_f16_to_f32((uint16_t)(p[0] | ((uint16_t)p[1] << 8)));
}

/* Rust `f32 as i32`: truncation toward zero, saturating, NaN -> 0 */
static int32_t f32_as_i32(float f) {
    if (f != f) {
        return 0;
    }
    if (f >= 2147483648.0f) {
        return INT32_MAX;
    }
    if (f <= -2147483648.0f) {
        return INT32_MIN;
    }
    return (int32_t)f;
}

static int32_t clampi(int32_t v, int32_t lo, int32_t hi) {
    return v < lo ? lo : (v > hi ? hi : v);
}

/* ---- quantizers, Q/quantize.rs ---- */

/* encode_q8_0_block, Q/quantize.rs:190-210 */
static void encode_q8_0_block(const float *values, uint8_t *out) {
    float amax = 0.0f;
    for (int i = 0; i < 32; i++) {
        amax = fmaxf(amax, fabsf(values[i])); /* acc.max(v.abs()), :194 */
    }
    float d = amax / 127.0f;                     /* :197 */
    float id = (d != 0.0f) ? 1.0f / d : 0.0f;    /* :198 */
    uint16_t h = oxq_ref_f32_to_f16(d);          /* :201 */
    out[0] = (uint8_t)(h & 0xFF);
    out[1] = (uint8_t)(h >> 8);
    for (int i = 0; i < 32; i++) {
        int32_t q = f32_as_i32(roundf(values[i] * id)); /* :206, round half away */
        out[2 + i] = (uint8_t)(int8_t)clampi(q, -128, 127); /* :207-208 */
    }
}

/* encode_q4_0_block, Q/quantize.rs:154-181 */
static void encode_q4_0_block(const float *values, uint8_t *out) {
    float max_val = 0.0f;
    for (int i = 0; i < 32; i++) {
        float v = values[i];
        if (fabsf(v) > fabsf(max_val)) { /* strict >, first wins, :161 */
            max_val = v;
        }
    }
    float d = max_val / -8.0f;                /* :164 */
    float id = (d != 0.0f) ? 1.0f / d : 0.0f; /* :165 */
    uint16_t h = oxq_ref_f32_to_f16(d);
    out[0] = (uint8_t)(h & 0xFF);
    out[1] = (uint8_t)(h >> 8);
    for (int pair = 0; pair < 16; pair++) {
        float x0 = values[pair * 2];
        float x1 = values[pair * 2 + 1];
        uint8_t q0 = (uint8_t)clampi(f32_as_i32(x0 * id + 8.5f), 0, 15); /* :176 */
        uint8_t q1 = (uint8_t)clampi(f32_as_i32(x1 * id + 8.5f), 0, 15); /* :177 */
        out[2 + pair] = (uint8_t)(q0 | (q1 << 4));                       /* :179 */
    }
}

/* quantize_f32_to_q8_0, Q/quantize.rs:58-75 */
oxq_ref_status oxq_ref_quantize_f32_to_q8_0(const float *x, size_t n, uint8_t *out) {
    if (n % 32 != 0) {
        return err(OXQ_REF_DIMENSION_MISMATCH, (n / 32 + 1) * 32, n);
    }
    for (size_t b = 0; b < n / 32; b++) {
        encode_q8_0_block(x + b * 32, out + b * 34);
    }
    return ok();
}

/* quantize_f32_to_q4_0, Q/quantize.rs:32-49 */
oxq_ref_status oxq_ref_quantize_f32_to_q4_0(const float *x, size_t n, uint8_t *out) {
    if (n % 32 != 0) {
        return err(OXQ_REF_DIMENSION_MISMATCH, (n / 32 + 1) * 32, n);
    }
    for (size_t b = 0; b < n / 32; b++) {
        encode_q4_0_block(x + b * 32, out + b * 18);
    }
    return ok();
}

/* ---- block decoders ---- */

/* decode_scales_mins, Q/reference/q4_k.rs:27-49 */
static void q4k_scales_mins(const uint8_t *s, uint8_t sc[8], uint8_t mn[8]) {
    for (int j = 0; j < 4; j++) {
        sc[j] = s[j] & 0x3F;
        mn[j] = s[j + 4] & 0x3F;
    }
    for (int j = 4; j < 8; j++) {
        uint8_t lo_sc = s[j + 4] & 0x0F;
        uint8_t hi_sc = (s[j - 4] >> 6) & 0x03;
        sc[j] = (uint8_t)(lo_sc | (hi_sc << 4));
        uint8_t lo_mn = (s[j + 4] >> 4) & 0x0F;
        uint8_t hi_mn = (s[j] >> 6) & 0x03;
        mn[j] = (uint8_t)(lo_mn | (hi_mn << 4));
    }
}

/* KVALUES_IQ4NL, Q/reference/iq_shared.rs:16-18 */
static const int8_t KVALUES_IQ4NL[16] = {-127, -104, -83, -65, -49, -35, -22, -10,
                                         1,    13,   25,  38,  53,  69,  89,  113};

/* unpack_sub_scale, Q/reference/iq4_xs.rs:47-53 */
static int32_t iq4xs_sub_scale(uint16_t scales_h, const uint8_t *scales_l, int i) {
    uint8_t ls_low = (uint8_t)((scales_l[i / 2] >> (4 * (i & 1))) & 0x0F);
    uint8_t ls_high = (uint8_t)((uint8_t)(scales_h >> (2 * i)) & 0x03);
    uint8_t ls = (uint8_t)(ls_low | (ls_high << 4));
    return (int32_t)ls - 32;
}

/* Q6_K: the four 6-bit quants (minus 32) decoded for index l of half `group`,
 * Q/reference/q6_k.rs:55-60 */
static void q6k_quads(const uint8_t *ql, const uint8_t *qh, int group, int l, int32_t q[4]) {
    int ql_off = group * 64, qh_off = group * 32;
    uint8_t h = qh[qh_off + l];
    q[0] = (int32_t)(uint8_t)((ql[ql_off + l] & 0x0F) | ((h & 3) << 4)) - 32;
    q[1] = (int32_t)(uint8_t)((ql[ql_off + l + 32] & 0x0F) | (((h >> 2) & 3) << 4)) - 32;
    q[2] = (int32_t)(uint8_t)((ql[ql_off + l] >> 4) | (((h >> 4) & 3) << 4)) - 32;
    q[3] = (int32_t)(uint8_t)((ql[ql_off + l + 32] >> 4) | (((h >> 6) & 3) << 4)) - 32;
}

static void dequant_q4_0(const uint8_t *block, float *out) {
    /* Q/reference/q4_0.rs:37-46 */
    float d = rd_f16(block);
    for (int i = 0; i < 16; i++) {
        uint8_t byte = block[2 + i];
        int32_t lo = (int32_t)(byte & 0x0F) - 8;
        int32_t hi = (int32_t)((byte >> 4) & 0x0F) - 8;
        out[i * 2] = (float)lo * d;
        out[i * 2 + 1] = (float)hi * d;
    }
}

static void dequant_q8_0(const uint8_t *block, float *out) {
    /* Q/reference/q8_0.rs:36-41 */
    float d = rd_f16(block);
    for (int i = 0; i < 32; i++) {
        out[i] = (float)(int8_t)block[2 + i] * d;
    }
}

static void dequant_q4_k(const uint8_t *block, float *out) {
    /* Q/reference/q4_k.rs:66-99 */
    float d = rd_f16(block);
    float dmin = rd_f16(block + 2);
    const uint8_t *qs = block + 16;
    uint8_t sc[8], mn[8];
    q4k_scales_mins(block + 4, sc, mn);
    int is = 0, qs_off = 0, out_off = 0;
    for (int g = 0; g < 4; g++) {
        float d1 = d * (float)sc[is];
        float m1 = dmin * (float)mn[is];
        float d2 = d * (float)sc[is + 1];
        float m2 = dmin * (float)mn[is + 1];
        for (int l = 0; l < 32; l++) {
            float q = (float)(qs[qs_off + l] & 0x0F);
            out[out_off + l] = d1 * q - m1;
        }
        for (int l = 0; l < 32; l++) {
            float q = (float)((qs[qs_off + l] >> 4) & 0x0F);
            out[out_off + 32 + l] = d2 * q - m2;
        }
        is += 2;
        qs_off += 32;
        out_off += 64;
    }
}

static void dequant_q6_k(const uint8_t *block, float *out) {
    /* Q/reference/q6_k.rs:39-72 */
    const uint8_t *ql = block, *qh = block + 128, *scales = block + 192;
    float d = rd_f16(block + 208);
    for (int group = 0; group < 2; group++) {
        int sc_off = group * 8, out_off = group * 128;
        for (int l = 0; l < 32; l++) {
            int is = l / 16;
            int32_t q[4];
            q6k_quads(ql, qh, group, l, q);
            float s0 = (float)(int8_t)scales[sc_off + is];
            float s1 = (float)(int8_t)scales[sc_off + is + 2];
            float s2 = (float)(int8_t)scales[sc_off + is + 4];
            float s3 = (float)(int8_t)scales[sc_off + is + 6];
            out[out_off + l] = d * s0 * (float)q[0];
            out[out_off + l + 32] = d * s1 * (float)q[1];
            out[out_off + l + 64] = d * s2 * (float)q[2];
            out[out_off + l + 96] = d * s3 * (float)q[3];
        }
    }
}

static void dequant_iq4_xs(const uint8_t *block, float *out) {
    /* Q/reference/iq4_xs.rs:73-94 */
    float d = rd_f16(block);
    uint16_t scales_h = (uint16_t)(block[2] | ((uint16_t)block[3] << 8));
    const uint8_t *scales_l = block + 4;
    const uint8_t *nibbles = block + 8;
    for (int sub = 0; sub < 8; sub++) {
        int32_t ls = iq4xs_sub_scale(scales_h, scales_l, sub);
        float scale = d * (float)ls;
        for (int i = 0; i < 16; i++) {
            uint8_t byte = nibbles[sub * 16 + i];
            out[sub * 32 + i * 2] = scale * (float)KVALUES_IQ4NL[byte & 0x0F];
            out[sub * 32 + i * 2 + 1] = scale * (float)KVALUES_IQ4NL[(byte >> 4) & 0x0F];
        }
    }
}

static void dequant_any(uint32_t type, const uint8_t *block, float *out) {
    switch (type) {
    case OXQ_REF_Q4_0:
        dequant_q4_0(block, out);
        break;
    case OXQ_REF_Q8_0:
        dequant_q8_0(block, out);
        break;
    case OXQ_REF_Q4_K:
        dequant_q4_k(block, out);
        break;
    case OXQ_REF_Q6_K:
        dequant_q6_k(block, out);
        break;
    case OXQ_REF_IQ4_XS:
        dequant_iq4_xs(block, out);
        break;
    default:
        oxq_more_dequant(type, block, out);
        break;
    }
}

/* dequant_block with the reference's checks (e.g. Q/reference/q4_k.rs:52-64) */
oxq_ref_status oxq_ref_dequant_block(uint32_t type, const uint8_t *block, size_t block_len,
                                     float *out, size_t out_len) {
    size_t bs = oxq_ref_block_size(type), bb = oxq_ref_block_bytes(type);
    if (bs == 0) {
        return err(OXQ_REF_UNSUPPORTED_TYPE, type, 0);
    }
    if (block_len < bb) {
        return err(OXQ_REF_BUFFER_TOO_SMALL, bb, block_len);
    }
    if (out_len < bs) {
        return err(OXQ_REF_BUFFER_TOO_SMALL, bs, out_len);
    }
    dequant_any(type, block, out);
    return ok();
}

/* ---- gemv (f32 activations), scalar tier ---- */

static float gemv_row_q4_0(const uint8_t *row, size_t bpr, size_t n_cols, const float *x) {
    /* Q/reference/q4_0.rs:82-102 */
    float sum = 0.0f;
    for (size_t blk = 0; blk < bpr; blk++) {
        const uint8_t *block = row + blk * 18;
        float d = rd_f16(block);
        size_t in_off = blk * 32;
        for (size_t i = 0; i < 16; i++) {
            uint8_t byte = block[2 + i];
            int32_t lo = (int32_t)(byte & 0x0F) - 8;
            int32_t hi = (int32_t)((byte >> 4) & 0x0F) - 8;
            size_t idx = in_off + i * 2;
            if (idx + 1 < n_cols) {
                sum += (float)lo * d * x[idx];
                sum += (float)hi * d * x[idx + 1];
            } else if (idx < n_cols) {
                sum += (float)lo * d * x[idx];
            }
        }
    }
    return sum;
}

static float gemv_row_q8_0(const uint8_t *row, size_t bpr, size_t n_cols, const float *x) {
    /* Q/reference/q8_0.rs:77-92 */
    float sum = 0.0f;
    for (size_t blk = 0; blk < bpr; blk++) {
        const uint8_t *block = row + blk * 34;
        float d = rd_f16(block);
        for (size_t i = 0; i < 32; i++) {
            size_t idx = blk * 32 + i;
            if (idx < n_cols) {
                sum += (float)(int8_t)block[2 + i] * d * x[idx];
            }
        }
    }
    return sum;
}

static float gemv_row_q4_k(const uint8_t *row, size_t bpr, size_t n_cols, const float *x) {
    /* Q/reference/q4_k.rs:135-178 */
    float sum = 0.0f;
    for (size_t blk = 0; blk < bpr; blk++) {
        const uint8_t *block = row + blk * 144;
        float d = rd_f16(block);
        float dmin = rd_f16(block + 2);
        const uint8_t *qs = block + 16;
        uint8_t sc[8], mn[8];
        q4k_scales_mins(block + 4, sc, mn);
        size_t is = 0, qs_off = 0, w_off = blk * 256;
        for (int g = 0; g < 4; g++) {
            float d1 = d * (float)sc[is];
            float m1 = dmin * (float)mn[is];
            float d2 = d * (float)sc[is + 1];
            float m2 = dmin * (float)mn[is + 1];
            for (size_t l = 0; l < 32; l++) {
                size_t idx = w_off + l;
                if (idx < n_cols) {
                    float q = (float)(qs[qs_off + l] & 0x0F);
                    sum += (d1 * q - m1) * x[idx];
                }
            }
            for (size_t l = 0; l < 32; l++) {
                size_t idx = w_off + 32 + l;
                if (idx < n_cols) {
                    float q = (float)((qs[qs_off + l] >> 4) & 0x0F);
                    sum += (d2 * q - m2) * x[idx];
                }
            }
            is += 2;
            qs_off += 32;
            w_off += 64;
        }
    }
    return sum;
}

static float gemv_row_q6_k(const uint8_t *row, size_t bpr, size_t n_cols, const float *x) {
    /* Q/reference/q6_k.rs:108-166 */
    float sum = 0.0f;
    for (size_t blk = 0; blk < bpr; blk++) {
        const uint8_t *b = row + blk * 210;
        const uint8_t *ql = b, *qh = b + 128, *scales = b + 192;
        float d = rd_f16(b + 208);
        const float *inp = x + blk * 256;
        size_t rem = n_cols - blk * 256;
        size_t cols_in_block = rem < 256 ? rem : 256;
        for (int group = 0; group < 2; group++) {
            int sc_off = group * 8;
            size_t in_off = (size_t)group * 128;
            for (int l = 0; l < 32; l++) {
                int is = l / 16;
                int32_t q[4];
                q6k_quads(ql, qh, group, l, q);
                float s0 = d * (float)(int8_t)scales[sc_off + is];
                float s1 = d * (float)(int8_t)scales[sc_off + is + 2];
                float s2 = d * (float)(int8_t)scales[sc_off + is + 4];
                float s3 = d * (float)(int8_t)scales[sc_off + is + 6];
                size_t c0 = in_off + (size_t)l, c1 = c0 + 32, c2 = c0 + 64, c3 = c0 + 96;
                if (c0 < cols_in_block) sum += s0 * (float)q[0] * inp[c0];
                if (c1 < cols_in_block) sum += s1 * (float)q[1] * inp[c1];
                if (c2 < cols_in_block) sum += s2 * (float)q[2] * inp[c2];
                if (c3 < cols_in_block) sum += s3 * (float)q[3] * inp[c3];
            }
        }
    }
    return sum;
}

static float gemv_row_iq4_xs(const uint8_t *row, size_t bpr, size_t n_cols, const float *x) {
    /* Q/reference/iq4_xs.rs:130-163 */
    float sum = 0.0f;
    for (size_t blk = 0; blk < bpr; blk++) {
        const uint8_t *block = row + blk * 136;
        float d = rd_f16(block);
        uint16_t scales_h = (uint16_t)(block[2] | ((uint16_t)block[3] << 8));
        const uint8_t *scales_l = block + 4;
        const uint8_t *nibbles = block + 8;
        for (int sub = 0; sub < 8; sub++) {
            int32_t ls = iq4xs_sub_scale(scales_h, scales_l, sub);
            float scale = d * (float)ls;
            size_t col_off = blk * 256 + (size_t)sub * 32;
            for (size_t i = 0; i < 16; i++) {
                uint8_t byte = nibbles[sub * 16 + i];
                size_t idx = col_off + i * 2;
                if (idx + 1 < n_cols) {
                    sum += (float)KVALUES_IQ4NL[byte & 0x0F] * scale * x[idx];
                    sum += (float)KVALUES_IQ4NL[(byte >> 4) & 0x0F] * scale * x[idx + 1];
                } else if (idx < n_cols) {
                    sum += (float)KVALUES_IQ4NL[byte & 0x0F] * scale * x[idx];
                }
            }
        }
    }
    return sum;
}

static float gemv_row(uint32_t type, const uint8_t *row, size_t bpr, size_t n_cols,
                      const float *x) {
    if (oxq_more_known(type)) {
        return oxq_more_gemv_row(type, row, bpr, n_cols, x);
    }
    switch (type) {
    case OXQ_REF_Q4_0:
        return gemv_row_q4_0(row, bpr, n_cols, x);
    case OXQ_REF_Q8_0:
        return gemv_row_q8_0(row, bpr, n_cols, x);
    case OXQ_REF_Q4_K:
        return gemv_row_q4_k(row, bpr, n_cols, x);
    case OXQ_REF_Q6_K:
        return gemv_row_q6_k(row, bpr, n_cols, x);
    default:
        return gemv_row_iq4_xs(row, bpr, n_cols, x);
    }
}

/* gemv with the reference's checks, e.g. Q/reference/q4_k.rs:104-184.  Output is
 * overwritten.  The reference slices `data[off..off+block_bytes]` and would panic
 * on a short buffer; here that is reported as BufferTooSmall. */
oxq_ref_status oxq_ref_gemv(uint32_t type, const uint8_t *w, size_t w_len, size_t n_rows,
                            size_t n_cols, const float *x, size_t x_len, float *y, size_t y_len) {
    size_t bs = oxq_ref_block_size(type), bb = oxq_ref_block_bytes(type);
    if (bs == 0) {
        return err(OXQ_REF_UNSUPPORTED_TYPE, type, 0);
    }
    if (x_len < n_cols) {
        return err(OXQ_REF_DIMENSION_MISMATCH, n_cols, x_len);
    }
    if (y_len < n_rows) {
        return err(OXQ_REF_DIMENSION_MISMATCH, n_rows, y_len);
    }
    size_t bpr = (n_cols + bs - 1) / bs;
    size_t row_bytes = bpr * bb;
    if (w_len < n_rows * row_bytes) {
        return err(OXQ_REF_BUFFER_TOO_SMALL, n_rows * row_bytes, w_len);
    }
    for (size_t r = 0; r < n_rows; r++) {
        y[r] = gemv_row(type, w + r * row_bytes, bpr, n_cols, x);
    }
    return ok();
}

/* gemm = m gemvs, Q/reference/q4_k.rs:186-201; x is [m x k], y is [m x n] */
oxq_ref_status oxq_ref_gemm(uint32_t type, const uint8_t *w, size_t w_len, const float *x,
                            float *y, size_t m, size_t n, size_t k) {
    for (size_t r = 0; r < m; r++) {
        oxq_ref_status s = oxq_ref_gemv(type, w, w_len, n, k, x + r * k, k, y + r * n, n);
        if (s.code != OXQ_REF_OK) {
            return s;
        }
    }
    return ok();
}

/* ---- matvec_q8_fused ---- */

/* Trait default, Q/traits.rs:137-170 (only valid for 32-weight blocks): dequantize
 * the weight block and the activation block to f32, multiply-accumulate. */
static float fused_row_default32(uint32_t type, const uint8_t *row, size_t bpr, size_t n_cols,
                                 const uint8_t *acts) {
    size_t bb = oxq_ref_block_bytes(type);
    float w_scratch[32], a_scratch[32];
    float sum = 0.0f;
    for (size_t blk = 0; blk < bpr; blk++) {
        dequant_any(type, row + blk * bb, w_scratch);
        const uint8_t *a_block = acts + blk * Q8_0_BLOCK_BYTES;
        float d_a = rd_f16(a_block);
        size_t w_start = blk * 32;
        size_t w_end = w_start + 32 < n_cols ? w_start + 32 : n_cols;
        size_t valid = w_end - w_start;
        for (size_t i = 0; i < valid; i++) {
            a_scratch[i] = (float)(int8_t)a_block[2 + i] * d_a;
        }
        for (size_t i = 0; i < valid; i++) {
            sum += w_scratch[i] * a_scratch[i];
        }
    }
    return sum;
}

/* matvec_q8_fused_reference, Q/reference/q4_0.rs:190-229 */
static float fused_row_q4_0_standalone(const uint8_t *row, size_t bpr, size_t n_cols,
                                       const uint8_t *acts) {
    float sum = 0.0f;
    for (size_t blk = 0; blk < bpr; blk++) {
        const uint8_t *w_block = row + blk * 18;
        float d_w = rd_f16(w_block);
        const uint8_t *a_block = acts + blk * Q8_0_BLOCK_BYTES;
        float d_a = rd_f16(a_block);
        const uint8_t *q8 = a_block + 2;
        size_t w_off = blk * 32;
        size_t valid = n_cols - w_off < 32 ? n_cols - w_off : 32;
        for (size_t i = 0; i < valid / 2; i++) {
            uint8_t byte = w_block[2 + i];
            int32_t q_lo = (int32_t)(byte & 0x0F) - 8;
            int32_t q_hi = (int32_t)((byte >> 4) & 0x0F) - 8;
            float a_lo = (float)(int8_t)q8[i * 2];
            float a_hi = (float)(int8_t)q8[i * 2 + 1];
            sum += (float)q_lo * d_w * a_lo * d_a;
            sum += (float)q_hi * d_w * a_hi * d_a;
        }
        if (valid % 2 == 1) {
            size_t i = valid / 2;
            uint8_t byte = w_block[2 + i];
            int32_t q_lo = (int32_t)(byte & 0x0F) - 8;
            float a_lo = (float)(int8_t)q8[i * 2];
            sum += (float)q_lo * d_w * a_lo * d_a;
        }
    }
    return sum;
}

/* fused_q4_0_q8_0_row_avx2, Q/simd/avx2/q4_0.rs:196-289: integer dot per block
 * (the lane order of the i32 horizontal sum is immaterial), one f32 term per block. */
static float fused_row_q4_0_avx2(const uint8_t *row, size_t bpr, size_t n_cols,
                                 const uint8_t *acts) {
    float row_sum = 0.0f;
    for (size_t blk = 0; blk < bpr; blk++) {
        const uint8_t *w_block = row + blk * 18;
        float d_w = rd_f16(w_block);
        const uint8_t *a_block = acts + blk * Q8_0_BLOCK_BYTES;
        float d_a = rd_f16(a_block);
        float scale = d_w * d_a; /* :211 */
        const uint8_t *q8 = a_block + 2;
        size_t in_off = blk * 32;
        size_t remaining = n_cols > in_off ? n_cols - in_off : 0;
        if (remaining >= 32) {
            int32_t dot = 0;
            for (int i = 0; i < 16; i++) {
                uint8_t byte = w_block[2 + i];
                dot += ((int32_t)(byte & 0x0F) - 8) * (int32_t)(int8_t)q8[2 * i];
                dot += ((int32_t)(byte >> 4) - 8) * (int32_t)(int8_t)q8[2 * i + 1];
            }
            row_sum += scale * (float)dot; /* :265 */
        } else if (remaining > 0) {
            size_t valid = remaining;
            for (size_t i = 0; i < valid / 2; i++) { /* :271-278 */
                uint8_t byte = w_block[2 + i];
                int32_t q_lo = (int32_t)(byte & 0x0F) - 8;
                int32_t q_hi = (int32_t)((byte >> 4) & 0x0F) - 8;
                int32_t a_lo = (int32_t)(int8_t)q8[i * 2];
                int32_t a_hi = (int32_t)(int8_t)q8[i * 2 + 1];
                row_sum += scale * (float)(q_lo * a_lo + q_hi * a_hi);
            }
            if (valid % 2 == 1) {
                size_t i = valid / 2;
                int32_t q_lo = (int32_t)(w_block[2 + i] & 0x0F) - 8;
                int32_t a_lo = (int32_t)(int8_t)q8[i * 2];
                row_sum += scale * (float)(q_lo * a_lo);
            }
        }
    }
    return row_sum;
}

/* fused_q8_0_q8_0_row_avx2, Q/simd/avx2/q8_0.rs:192-255 */
static float fused_row_q8_0_avx2(const uint8_t *row, size_t bpr, size_t n_cols,
                                 const uint8_t *acts) {
    float row_sum = 0.0f;
    for (size_t blk = 0; blk < bpr; blk++) {
        const uint8_t *w_block = row + blk * 34;
        float d_w = rd_f16(w_block);
        const uint8_t *a_block = acts + blk * 34;
        float d_a = rd_f16(a_block);
        float scale = d_w * d_a; /* :205 */
        size_t in_off = blk * 32;
        size_t remaining = n_cols > in_off ? n_cols - in_off : 0;
        if (remaining >= 32) {
            int32_t dot = 0;
            for (int i = 0; i < 32; i++) {
                dot += (int32_t)(int8_t)w_block[2 + i] * (int32_t)(int8_t)a_block[2 + i];
            }
            row_sum += scale * (float)dot; /* :242 */
        } else if (remaining > 0) {
            float partial = 0.0f; /* :247-251 */
            for (size_t i = 0; i < remaining; i++) {
                partial += (float)(int8_t)w_block[2 + i] * (float)(int8_t)a_block[2 + i];
            }
            row_sum += scale * partial;
        }
    }
    return row_sum;
}

/* One Q4_K super-block against its 8 activation blocks in the scalar-tier order
 * (Q/reference/q4_k.rs:272-326): eight terms, each added straight into *sum. */
static void fused_q4k_block_scalar(const uint8_t *block, const uint8_t *acts, size_t blk,
                                   size_t n_cols, float *sum) {
    float d = rd_f16(block);
    float dmin = rd_f16(block + 2);
    uint8_t sc[8], mn[8];
    q4k_scales_mins(block + 4, sc, mn);
    const uint8_t *qs = block + 16;
    size_t is = 0, qs_off = 0, w_off = blk * 256;
    for (int g = 0; g < 4; g++) {
        const uint8_t *a_lo = acts + (blk * 8 + is) * Q8_0_BLOCK_BYTES;
        const uint8_t *a_hi = acts + (blk * 8 + is + 1) * Q8_0_BLOCK_BYTES;
        float d_a_lo = rd_f16(a_lo), d_a_hi = rd_f16(a_hi);
        float da_lo = d * (float)sc[is];
        float m_lo = dmin * (float)mn[is];
        float da_hi = d * (float)sc[is + 1];
        float m_hi = dmin * (float)mn[is + 1];
        float dot_lo = 0.0f, sum_a_lo = 0.0f;
        for (size_t l = 0; l < 32; l++) {
            if (w_off + l < n_cols) {
                float q_w = (float)(qs[qs_off + l] & 0x0F);
                float q_a = (float)(int8_t)a_lo[2 + l];
                dot_lo += q_w * q_a;
                sum_a_lo += q_a;
            }
        }
        *sum += (da_lo * dot_lo - m_lo * sum_a_lo) * d_a_lo; /* :307 */
        float dot_hi = 0.0f, sum_a_hi = 0.0f;
        for (size_t l = 0; l < 32; l++) {
            if (w_off + 32 + l < n_cols) {
                float q_w = (float)((qs[qs_off + l] >> 4) & 0x0F);
                float q_a = (float)(int8_t)a_hi[2 + l];
                dot_hi += q_w * q_a;
                sum_a_hi += q_a;
            }
        }
        *sum += (da_hi * dot_hi - m_hi * sum_a_hi) * d_a_hi; /* :321 */
        is += 2;
        qs_off += 32;
        w_off += 64;
    }
}

/* Q4KRef::matvec_q8_fused row, Q/reference/q4_k.rs:252-330 */
static float fused_row_q4_k_scalar(const uint8_t *row, size_t bpr, size_t n_cols,
                                   const uint8_t *acts) {
    float sum = 0.0f;
    for (size_t blk = 0; blk < bpr; blk++) {
        fused_q4k_block_scalar(row + blk * 144, acts, blk, n_cols, &sum);
    }
    return sum;
}

/* fused_q4k_q8_0_row_avx2, Q/simd/avx2/q4_k.rs:233-433: integer dot and integer
 * activation sum per sub-block, eight terms summed into block_sum, then row_sum. */
static float fused_row_q4_k_avx2(const uint8_t *row, size_t bpr, size_t n_cols,
                                 const uint8_t *acts) {
    float row_sum = 0.0f;
    for (size_t blk = 0; blk < bpr; blk++) {
        const uint8_t *block = row + blk * 144;
        size_t in_off = blk * 256;
        size_t remaining = n_cols > in_off ? n_cols - in_off : 0;
        if (remaining >= 256) {
            float d = rd_f16(block);
            float dmin = rd_f16(block + 2);
            uint8_t sc[8], mn[8];
            q4k_scales_mins(block + 4, sc, mn);
            const uint8_t *qs = block + 16;
            float block_sum = 0.0f;
            size_t is = 0, qs_off = 0;
            for (int g = 0; g < 4; g++) {
                const uint8_t *a_lo = acts + (blk * 8 + is) * Q8_0_BLOCK_BYTES;
                const uint8_t *a_hi = acts + (blk * 8 + is + 1) * Q8_0_BLOCK_BYTES;
                float d_a_lo = rd_f16(a_lo), d_a_hi = rd_f16(a_hi);
                float da_lo = d * (float)sc[is];
                float m_lo = dmin * (float)mn[is];
                float da_hi = d * (float)sc[is + 1];
                float m_hi = dmin * (float)mn[is + 1];
                int32_t dot_lo = 0, sum_a_lo = 0, dot_hi = 0, sum_a_hi = 0;
                for (int l = 0; l < 32; l++) {
                    int32_t qa = (int32_t)(int8_t)a_lo[2 + l];
                    dot_lo += (int32_t)(qs[qs_off + l] & 0x0F) * qa;
                    sum_a_lo += qa;
                    int32_t qb = (int32_t)(int8_t)a_hi[2 + l];
                    dot_hi += (int32_t)(qs[qs_off + l] >> 4) * qb;
                    sum_a_hi += qb;
                }
                block_sum += (da_lo * (float)dot_lo - m_lo * (float)sum_a_lo) * d_a_lo; /* :329 */
                block_sum += (da_hi * (float)dot_hi - m_hi * (float)sum_a_hi) * d_a_hi; /* :361 */
                is += 2;
                qs_off += 32;
            }
            row_sum += block_sum; /* :367 */
        } else if (remaining > 0) {
            float partial = 0.0f; /* scalar tail :370-428 */
            fused_q4k_block_scalar(block, acts, blk, n_cols, &partial);
            row_sum += partial;
        }
    }
    return row_sum;
}

/* Q6KRef::matvec_q8_fused row, Q/reference/q6_k.rs:246-351; the AVX2 tier's body
 * (Q/simd/avx2/q6_k.rs:208-283) is the same scalar code. */
static float fused_row_q6_k(const uint8_t *row, size_t bpr, size_t n_cols, const uint8_t *acts) {
    float sum = 0.0f;
    for (size_t blk = 0; blk < bpr; blk++) {
        const uint8_t *b = row + blk * 210;
        const uint8_t *ql = b, *qh = b + 128, *scales = b + 192;
        float d = rd_f16(b + 208);
        size_t in_base = blk * 256;
        size_t cols_in_block = n_cols - in_base < 256 ? n_cols - in_base : 256;
        for (int group = 0; group < 2; group++) {
            int sc_off = group * 8;
            size_t in_off = (size_t)group * 128;
            for (int l = 0; l < 32; l++) {
                int is = l / 16;
                int32_t q[4];
                q6k_quads(ql, qh, group, l, q);
                float s[4];
                for (int j = 0; j < 4; j++) {
                    s[j] = d * (float)(int8_t)scales[sc_off + is + 2 * j];
                }
                for (int j = 0; j < 4; j++) {
                    size_t col = in_off + (size_t)l + 32 * (size_t)j;
                    if (col < cols_in_block) {
                        const uint8_t *ab = acts + (blk * 8 + col / 32) * Q8_0_BLOCK_BYTES;
                        float d_a = rd_f16(ab);
                        float q_a = (float)(int8_t)ab[2 + col % 32];
                        float a = d_a * q_a;            /* :331 */
                        sum += s[j] * (float)q[j] * a; /* :335-344 */
                    }
                }
            }
        }
    }
    return sum;
}

/* ---- integer sums per group (32 weights; 16 for Q6_K) ---- */

static void block_sums_row(uint32_t type, const uint8_t *row, size_t bpr, const uint8_t *acts,
                           int32_t *sums) {
    if (oxq_more_known(type)) {
        oxq_more_block_sums_row(type, row, bpr, acts, sums);
        return;
    }
    switch (type) {
    case OXQ_REF_Q4_0:
        for (size_t blk = 0; blk < bpr; blk++) {
            const uint8_t *w = row + blk * 18 + 2;
            const uint8_t *a = acts + blk * 34 + 2;
            int32_t s = 0;
            for (int i = 0; i < 16; i++) {
                s += ((int32_t)(w[i] & 0x0F) - 8) * (int32_t)(int8_t)a[2 * i];
                s += ((int32_t)(w[i] >> 4) - 8) * (int32_t)(int8_t)a[2 * i + 1];
            }
            sums[blk] = s;
        }
        break;
    case OXQ_REF_Q8_0:
        for (size_t blk = 0; blk < bpr; blk++) {
            const uint8_t *w = row + blk * 34 + 2;
            const uint8_t *a = acts + blk * 34 + 2;
            int32_t s = 0;
            for (int i = 0; i < 32; i++) {
                s += (int32_t)(int8_t)w[i] * (int32_t)(int8_t)a[i];
            }
            sums[blk] = s;
        }
        break;
    case OXQ_REF_Q4_K:
        for (size_t blk = 0; blk < bpr; blk++) {
            const uint8_t *qs = row + blk * 144 + 16;
            for (int g = 0; g < 4; g++) {
                const uint8_t *a_lo = acts + (blk * 8 + 2 * g) * 34 + 2;
                const uint8_t *a_hi = acts + (blk * 8 + 2 * g + 1) * 34 + 2;
                int32_t lo = 0, hi = 0;
                for (int l = 0; l < 32; l++) {
                    lo += (int32_t)(qs[32 * g + l] & 0x0F) * (int32_t)(int8_t)a_lo[l];
                    hi += (int32_t)(qs[32 * g + l] >> 4) * (int32_t)(int8_t)a_hi[l];
                }
                sums[blk * 8 + 2 * g] = lo;
                sums[blk * 8 + 2 * g + 1] = hi;
            }
        }
        break;
    case OXQ_REF_Q6_K:
        for (size_t blk = 0; blk < bpr; blk++) {
            const uint8_t *b = row + blk * 210;
            int32_t *out = sums + blk * 16;
            for (int i = 0; i < 16; i++) {
                out[i] = 0;
            }
            for (int group = 0; group < 2; group++) {
                for (int l = 0; l < 32; l++) {
                    int32_t q[4];
                    q6k_quads(b, b + 128, group, l, q);
                    for (int j = 0; j < 4; j++) {
                        int col = group * 128 + l + 32 * j;
                        const uint8_t *ab = acts + (blk * 8 + (size_t)col / 32) * 34;
                        out[col / 16] += q[j] * (int32_t)(int8_t)ab[2 + col % 32];
                    }
                }
            }
        }
        break;
    default: /* IQ4_XS */
        for (size_t blk = 0; blk < bpr; blk++) {
            const uint8_t *nib = row + blk * 136 + 8;
            for (int sub = 0; sub < 8; sub++) {
                const uint8_t *a = acts + (blk * 8 + sub) * 34 + 2;
                int32_t s = 0;
                for (int i = 0; i < 16; i++) {
                    uint8_t byte = nib[sub * 16 + i];
                    s += (int32_t)KVALUES_IQ4NL[byte & 0x0F] * (int32_t)(int8_t)a[2 * i];
                    s += (int32_t)KVALUES_IQ4NL[byte >> 4] * (int32_t)(int8_t)a[2 * i + 1];
                }
                sums[blk * 8 + sub] = s;
            }
        }
        break;
    }
}

static size_t groups_per_block(uint32_t type) {
    if (oxq_more_known(type)) {
        return oxq_more_groups_per_block(type);
    }
    switch (type) {
    case OXQ_REF_Q6_K:
        return 16;
    case OXQ_REF_Q4_K:
    case OXQ_REF_IQ4_XS:
        return 8;
    default:
        return 1;
    }
}

/* Integer-dot row in the canonical order of the fused kernels: group terms left
 * to right, each an fp32 product of scales with the exact integer sum.
 *   Q4_0, Q8_0 : (d_w*d_a) * float(isum)                    (AVX2 tier, exact twin)
 *   Q4_K       : (d*sc*float(isum) - dmin*mn*float(asum))*d_a, eight terms into a
 *                per-super-block partial                     (AVX2 tier, exact twin)
 *   Q6_K       : (d*sc) * float(isum16) * d_a  per 16 weights
 *   IQ4_XS     : (d*ls) * float(isum) * d_a    per 32 weights
 */
static float intdot_row(uint32_t type, const uint8_t *row, size_t bpr, size_t n_cols,
                        const uint8_t *acts, int32_t *scratch) {
    if (oxq_more_known(type)) {
        return oxq_more_intdot_row(type, row, bpr, acts, scratch);
    }
    switch (type) {
    case OXQ_REF_Q4_0:
        return fused_row_q4_0_avx2(row, bpr, n_cols, acts);
    case OXQ_REF_Q8_0:
        return fused_row_q8_0_avx2(row, bpr, n_cols, acts);
    case OXQ_REF_Q4_K:
        return fused_row_q4_k_avx2(row, bpr, n_cols, acts);
    case OXQ_REF_Q6_K: {
        block_sums_row(type, row, bpr, acts, scratch);
        float sum = 0.0f;
        for (size_t blk = 0; blk < bpr; blk++) {
            const uint8_t *b = row + blk * 210;
            float d = rd_f16(b + 208);
            for (int g = 0; g < 16; g++) {
                float d_a = rd_f16(acts + (blk * 8 + (size_t)g / 2) * 34);
                float s = d * (float)(int8_t)b[192 + g];
                sum += s * (float)scratch[blk * 16 + g] * d_a;
            }
        }
        return sum;
    }
    default: {
        block_sums_row(type, row, bpr, acts, scratch);
        float sum = 0.0f;
        for (size_t blk = 0; blk < bpr; blk++) {
            const uint8_t *b = row + blk * 136;
            float d = rd_f16(b);
            uint16_t scales_h = (uint16_t)(b[2] | ((uint16_t)b[3] << 8));
            for (int sub = 0; sub < 8; sub++) {
                float d_a = rd_f16(acts + (blk * 8 + (size_t)sub) * 34);
                float scale = d * (float)iq4xs_sub_scale(scales_h, b + 4, sub);
                sum += scale * (float)scratch[blk * 8 + sub] * d_a;
            }
        }
        return sum;
    }
    }
}

/* Validation shared by every fused entry point, in the reference's order
 * (Q/reference/q4_k.rs:226-250; Q/traits.rs:99-130). */
static oxq_ref_status fused_validate(uint32_t type, size_t w_len, size_t acts_len, size_t out_len,
                                     size_t n_rows, size_t n_cols, size_t *bpr_out) {
    size_t bs = oxq_ref_block_size(type), bb = oxq_ref_block_bytes(type);
    if (bs == 0) {
        return err(OXQ_REF_UNSUPPORTED_TYPE, type, 0);
    }
    if (out_len < n_rows) {
        return err(OXQ_REF_DIMENSION_MISMATCH, n_rows, out_len);
    }
    size_t bpr = (n_cols + bs - 1) / bs;
    size_t row_bytes = bpr * bb;
    size_t acts_needed = bpr * (bs / 32) * Q8_0_BLOCK_BYTES;
    if (w_len < n_rows * row_bytes) {
        return err(OXQ_REF_BUFFER_TOO_SMALL, n_rows * row_bytes, w_len);
    }
    if (acts_len < acts_needed) {
        return err(OXQ_REF_BUFFER_TOO_SMALL, acts_needed, acts_len);
    }
    *bpr_out = bpr;
    return ok();
}

static float fused_row(uint32_t type, int tier, const uint8_t *row, size_t bpr, size_t n_cols,
                       const uint8_t *acts, int32_t *scratch) {
    if (oxq_more_known(type)) { /* one tier: the *Ref kernels of Q/reference */
        return oxq_more_fused_row(type, row, bpr, n_cols, acts);
    }
    switch (type) {
    case OXQ_REF_Q4_0:
        if (tier == OXQ_REF_TIER_AVX2) return fused_row_q4_0_avx2(row, bpr, n_cols, acts);
        if (tier == OXQ_REF_TIER_Q4_0_STANDALONE)
            return fused_row_q4_0_standalone(row, bpr, n_cols, acts);
        return fused_row_default32(type, row, bpr, n_cols, acts);
    case OXQ_REF_Q8_0:
        if (tier == OXQ_REF_TIER_AVX2) return fused_row_q8_0_avx2(row, bpr, n_cols, acts);
        return fused_row_default32(type, row, bpr, n_cols, acts);
    case OXQ_REF_Q4_K:
        if (tier == OXQ_REF_TIER_AVX2) return fused_row_q4_k_avx2(row, bpr, n_cols, acts);
        return fused_row_q4_k_scalar(row, bpr, n_cols, acts);
    case OXQ_REF_Q6_K:
        return fused_row_q6_k(row, bpr, n_cols, acts);
    default:
        /* IQ4_XS: no working reference kernel; integer form defined by this build */
        return intdot_row(type, row, bpr, n_cols, acts, scratch);
    }
}

oxq_ref_status oxq_ref_matvec_q8_fused(uint32_t type, int tier, const uint8_t *w, size_t w_len,
                                       const uint8_t *acts, size_t acts_len, float *out,
                                       size_t out_len, size_t n_rows, size_t n_cols) {
    size_t bpr = 0;
    oxq_ref_status s = fused_validate(type, w_len, acts_len, out_len, n_rows, n_cols, &bpr);
    if (s.code != OXQ_REF_OK) {
        return s;
    }
    if (type == OXQ_REF_IQ4_XS && n_cols % 256 != 0) {
        return err(OXQ_REF_KERNEL_ERROR, n_cols, 256);
    }
    size_t row_bytes = bpr * oxq_ref_block_bytes(type);
    int32_t *scratch = (int32_t *)malloc(sizeof(int32_t) * (bpr * 16 + 16));
    if (!scratch) {
        return err(OXQ_REF_INTERNAL, 0, 0);
    }
    for (size_t r = 0; r < n_rows; r++) {
        out[r] += fused_row(type, tier, w + r * row_bytes, bpr, n_cols, acts, scratch); /* ACCUMULATE */
    }
    free(scratch);
    return ok();
}

oxq_ref_status oxq_ref_matvec_q8_intdot(uint32_t type, const uint8_t *w, size_t w_len,
                                        const uint8_t *acts, size_t acts_len, float *out,
                                        size_t out_len, size_t n_rows, size_t n_cols) {
    size_t bpr = 0;
    oxq_ref_status s = fused_validate(type, w_len, acts_len, out_len, n_rows, n_cols, &bpr);
    if (s.code != OXQ_REF_OK) {
        return s;
    }
    if ((type == OXQ_REF_IQ4_XS || type == OXQ_REF_Q6_K || oxq_more_known(type)) &&
        n_cols % oxq_ref_block_size(type) != 0) {
        return err(OXQ_REF_KERNEL_ERROR, n_cols, oxq_ref_block_size(type));
    }
    size_t row_bytes = bpr * oxq_ref_block_bytes(type);
    int32_t *scratch = (int32_t *)malloc(sizeof(int32_t) * (bpr * 16 + 16));
    if (!scratch) {
        return err(OXQ_REF_INTERNAL, 0, 0);
    }
    for (size_t r = 0; r < n_rows; r++) {
        out[r] += intdot_row(type, w + r * row_bytes, bpr, n_cols, acts, scratch);
    }
    free(scratch);
    return ok();
}

oxq_ref_status oxq_ref_block_sums(uint32_t type, const uint8_t *w, size_t w_len,
                                  const uint8_t *acts, size_t acts_len, int32_t *sums,
                                  size_t n_rows, size_t n_cols) {
    size_t bpr = 0;
    oxq_ref_status s = fused_validate(type, w_len, acts_len, n_rows, n_rows, n_cols, &bpr);
    if (s.code != OXQ_REF_OK) {
        return s;
    }
    if (n_cols % oxq_ref_block_size(type) != 0) {
        return err(OXQ_REF_KERNEL_ERROR, n_cols, oxq_ref_block_size(type));
    }
    size_t row_bytes = bpr * oxq_ref_block_bytes(type);
    size_t gpr = bpr * groups_per_block(type);
    for (size_t r = 0; r < n_rows; r++) {
        block_sums_row(type, w + r * row_bytes, bpr, acts, sums + r * gpr);
    }
    return ok();
}

oxq_ref_status oxq_ref_gemm_q8(uint32_t type, int tier, const uint8_t *w, size_t w_len,
                               const float *x, float *y, size_t m, size_t n, size_t k) {
    size_t bs = oxq_ref_block_size(type);
    if (bs == 0) {
        return err(OXQ_REF_UNSUPPORTED_TYPE, type, 0);
    }
    if (k % 32 != 0) {
        return err(OXQ_REF_DIMENSION_MISMATCH, (k / 32 + 1) * 32, k);
    }
    size_t bpr = (k + bs - 1) / bs;
    size_t acts_len = bpr * (bs / 32) * Q8_0_BLOCK_BYTES;
    uint8_t *acts = (uint8_t *)calloc(acts_len, 1);
    if (!acts) {
        return err(OXQ_REF_INTERNAL, 0, 0);
    }
    oxq_ref_status s = ok();
    for (size_t r = 0; r < m && s.code == OXQ_REF_OK; r++) {
        s = oxq_ref_quantize_f32_to_q8_0(x + r * k, k, acts);
        if (s.code != OXQ_REF_OK) {
            break;
        }
        memset(y + r * n, 0, n * sizeof(float));
        s = oxq_ref_matvec_q8_fused(type, tier, w, w_len, acts, acts_len, y + r * n, n, n, k);
    }
    free(acts);
    return s;
}

/* ---- threaded row split (CPU baseline timing only), Q/parallel.rs:70-77 ---- */
#include <pthread.h>

typedef struct {
    uint32_t type;
    int tier;
    const uint8_t *w;
    const uint8_t *acts;
    float *out;
    size_t row0, row1, bpr, n_cols, row_bytes;
} mt_job;

static void *mt_worker(void *p) {
    mt_job *j = (mt_job *)p;
    int32_t *scratch = (int32_t *)malloc(sizeof(int32_t) * (j->bpr * 16 + 16));
    for (size_t r = j->row0; r < j->row1; r++) {
        j->out[r] += fused_row(j->type, j->tier, j->w + r * j->row_bytes, j->bpr, j->n_cols,
                               j->acts, scratch);
    }
    free(scratch);
    return NULL;
}

oxq_ref_status oxq_ref_matvec_q8_fused_mt(uint32_t type, int tier, const uint8_t *w, size_t w_len,
                                          const uint8_t *acts, size_t acts_len, float *out,
                                          size_t out_len, size_t n_rows, size_t n_cols,
                                          int n_threads) {
    size_t bpr = 0;
    oxq_ref_status s = fused_validate(type, w_len, acts_len, out_len, n_rows, n_cols, &bpr);
    if (s.code != OXQ_REF_OK) {
        return s;
    }
    if (n_threads < 1) {
        n_threads = 1;
    }
    if (n_threads > 256) {
        n_threads = 256;
    }
    pthread_t th[256];
    mt_job jobs[256];
    size_t chunk = (n_rows + (size_t)n_threads - 1) / (size_t)n_threads;
    int started = 0;
    for (int t = 0; t < n_threads; t++) {
        size_t r0 = (size_t)t * chunk;
        if (r0 >= n_rows) {
            break;
        }
        size_t r1 = r0 + chunk < n_rows ? r0 + chunk : n_rows;
        mt_job j = {type, tier, w, acts, out, r0, r1, bpr, n_cols, bpr * oxq_ref_block_bytes(type)};
        jobs[t] = j;
        if (pthread_create(&th[t], NULL, mt_worker, &jobs[t]) != 0) {
            mt_worker(&jobs[t]);
            th[t] = 0;
        }
        started = t + 1;
    }
    for (int t = 0; t < started; t++) {
        if (th[t]) {
            pthread_join(th[t], NULL);
        }
    }
    return ok();
}
