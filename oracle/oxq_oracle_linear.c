/*
 * oxq_oracle_linear.c -- TEST INFRASTRUCTURE, NOT PRODUCT CODE.
 *
 * Scalar C restatement of the callers' glue around the quantized matvec in the reference
 * (/root/reference): SwiGLU, RMSNorm, the LoRA correction and QuantLinear::forward.  Same
 * rules as oxq_oracle.c: reference operation order, -ffp-contract=off -fno-fast-math.
 *
 * Pinning (tests/test_oracle_linear.py):
 *   swiglu_inplace     the reference's own values (swiglu.rs:62-77) and a float64 closed form
 *   rmsnorm_forward_to the reference's tests (rms_norm.rs:72-127) and a float64 closed form
 *   lora_apply         the reference's hand-computed cases (lora.rs:141-200) and its error
 *                      cases (lora.rs:229-259); float64 recomputation on random adapters
 *   linear_forward     the reference's QuantLinear tests (linear.rs:161-270) replayed on Q8_0
 *                      tensors with exactly representable weights
 */
#include <math.h>
#include <stdlib.h>
#include <string.h>

#include "oxq_oracle.h"

static oxq_ref_status st(int code, size_t a, size_t b) {
    oxq_ref_status s = {code, a, b};
    return s;
}

/* swiglu_inplace, crates/oxillama-arch/src/common/swiglu.rs:15-21 */
void oxq_ref_swiglu_inplace(float *gate, const float *up, size_t n) {
    for (size_t i = 0; i < n; i++) {
        float g = gate[i];
        float sigmoid = 1.0f / (1.0f + expf(-g)); /* :18 */
        gate[i] = g * sigmoid * up[i];            /* :19, (g * sigmoid) * u */
    }
}

/* RmsNorm::forward_to, crates/oxillama-arch/src/common/rms_norm.rs:49-66 */
void oxq_ref_rmsnorm_forward_to(const float *input, const float *weight, float eps, size_t n,
                                float *output) {
    if (n == 0) {
        return;
    }
    float sum_sq = 0.0f;
    for (size_t i = 0; i < n; i++) {
        sum_sq += input[i] * input[i]; /* :56-58, index order */
    }
    float rms = sqrtf(sum_sq / (float)n + eps); /* :59 */
    float inv_rms = 1.0f / rms;                 /* :60 */
    for (size_t i = 0; i < n; i++) {
        output[i] = input[i] * inv_rms * weight[i]; /* :63 */
    }
}

/* LoraAdapter::new, crates/oxillama-quant/src/lora.rs:43-73: size checks only */
oxq_ref_status oxq_ref_lora_new(size_t a_len, size_t b_len, size_t rank, size_t in_features,
                                size_t out_features) {
    if (a_len != rank * in_features) {
        return st(OXQ_REF_DIMENSION_MISMATCH, rank * in_features, a_len);
    }
    if (b_len != out_features * rank) {
        return st(OXQ_REF_DIMENSION_MISMATCH, out_features * rank, b_len);
    }
    return st(OXQ_REF_OK, 0, 0);
}

/* LoraAdapter::apply, crates/oxillama-quant/src/lora.rs:83-124.  Both sums are Rust iterator
 * sums: a left fold from 0.0 in index order. */
oxq_ref_status oxq_ref_lora_apply(const float *a, const float *b, size_t rank, float scale,
                                  size_t in_features, size_t out_features, const float *input,
                                  size_t input_len, float *output, size_t output_len) {
    if (input_len < in_features) {
        return st(OXQ_REF_DIMENSION_MISMATCH, in_features, input_len);
    }
    if (output_len < out_features) {
        return st(OXQ_REF_DIMENSION_MISMATCH, out_features, output_len);
    }
    float *r_vec = (float *)calloc(rank ? rank : 1, sizeof(float));
    if (!r_vec) {
        return st(OXQ_REF_INTERNAL, 0, 0);
    }
    for (size_t i = 0; i < rank; i++) {
        const float *row = a + i * in_features;
        float s = 0.0f;
        for (size_t j = 0; j < in_features; j++) {
            s += row[j] * input[j];
        }
        r_vec[i] = s;
    }
    for (size_t i = 0; i < out_features; i++) {
        const float *row = b + i * rank;
        float s = 0.0f;
        for (size_t j = 0; j < rank; j++) {
            s += row[j] * r_vec[j];
        }
        float delta = s * scale; /* :114-119 */
        output[i] += delta;      /* :120 */
    }
    free(r_vec);
    return st(OXQ_REF_OK, 0, 0);
}

/* QuantLinear::forward, crates/oxillama-arch/src/common/linear.rs:77-98, with `gemv` taken on
 * the Q8_0-activation path this build accelerates (quantize the input, fused matvec into a
 * zeroed output), then bias (zip: the shorter of the two lengths), then LoRA. */
oxq_ref_status oxq_ref_linear_forward(uint32_t type, int tier, const uint8_t *w, size_t w_len,
                                      size_t n_rows, size_t n_cols, const float *bias, size_t bias_len,
                                      const float *lora_a, const float *lora_b, size_t rank, float scale,
                                      const float *input, size_t input_len, float *output,
                                      size_t output_len) {
    if (input_len < n_cols) {
        return st(OXQ_REF_DIMENSION_MISMATCH, n_cols, input_len); /* gemv's checks, q4_k.rs:117-128 */
    }
    if (output_len < n_rows) {
        return st(OXQ_REF_DIMENSION_MISMATCH, n_rows, output_len);
    }
    /* A row that ends inside a block: the reference's gemv skips the columns past n_cols
     * (q4_k.rs:161,168); with Q8_0 activations that is the input zero-padded to whole blocks. */
    size_t bs = oxq_ref_block_size(type);
    if (bs == 0) {
        return st(OXQ_REF_UNSUPPORTED_TYPE, type, 0);
    }
    size_t k_pad = (n_cols + bs - 1) / bs * bs;
    size_t acts_len = k_pad / 32 * 34;
    uint8_t *acts = (uint8_t *)malloc(acts_len ? acts_len : 1);
    float *padded = (float *)calloc(k_pad ? k_pad : 1, sizeof(float));
    if (!acts || !padded) {
        free(acts);
        free(padded);
        return st(OXQ_REF_INTERNAL, 0, 0);
    }
    memcpy(padded, input, n_cols * sizeof(float));
    oxq_ref_status s = oxq_ref_quantize_f32_to_q8_0(padded, k_pad, acts);
    free(padded);
    if (s.code == OXQ_REF_OK) {
        for (size_t r = 0; r < n_rows; r++) {
            output[r] = 0.0f; /* gemv overwrites */
        }
        s = oxq_ref_matvec_q8_fused(type, tier, w, w_len, acts, acts_len, output, output_len, n_rows, n_cols);
    }
    free(acts);
    if (s.code != OXQ_REF_OK) {
        return s;
    }
    if (bias) {
        size_t nb = bias_len < n_rows ? bias_len : n_rows; /* :87-89 */
        for (size_t i = 0; i < nb; i++) {
            output[i] += bias[i];
        }
    }
    if (lora_a && lora_b && rank) {
        return oxq_ref_lora_apply(lora_a, lora_b, rank, scale, n_cols, n_rows, input, input_len, output,
                                  output_len); /* :93-95 */
    }
    return st(OXQ_REF_OK, 0, 0);
}

/* argmax, crates/oxillama-runtime/src/sampling/mod.rs:652-662: strict '>' from -inf, so the first of
 * equal maxima wins (and index 0 when nothing exceeds -inf). */
uint32_t oxq_ref_argmax(const float *values, size_t n) {
    uint32_t max_idx = 0;
    float max_val = -INFINITY;
    for (size_t i = 0; i < n; i++) {
        if (values[i] > max_val) {
            max_val = values[i];
            max_idx = (uint32_t)i;
        }
    }
    return max_idx;
}

/* The sampler's candidate list, mod.rs:500-509: (index, value) pairs sorted by value, largest first,
 * truncated to k.  The reference's sort_unstable_by leaves the order of equal values open; this
 * restatement fixes it (lower index first) and ranks NaN last.  O(n k) selection, small inputs only. */
void oxq_ref_topk(const float *values, size_t n, size_t k, float *out_vals, uint32_t *out_idx) {
    unsigned char *taken = (unsigned char *)calloc(n ? n : 1, 1);
    for (size_t r = 0; r < k && r < n; r++) {
        size_t best = n;
        for (size_t i = 0; i < n; i++) {
            if (taken[i]) {
                continue;
            }
            if (best == n) {
                best = i;
                continue;
            }
            float a = values[i], b = values[best];
            int a_nan = a != a, b_nan = b != b;
            if ((b_nan && !a_nan) || (!a_nan && !b_nan && a > b)) {
                best = i;
            }
        }
        taken[best] = 1;
        out_vals[r] = values[best];
        out_idx[r] = (uint32_t)best;
    }
    free(taken);
}

/* Xorshift64, sampling/mod.rs:669-690 */
uint64_t oxq_ref_xorshift64_seed(uint64_t seed) { return seed == 0 ? 0x517cc1b727220a95ull : seed; }

float oxq_ref_xorshift64_next_f32(uint64_t *state) {
    uint64_t x = *state;
    x ^= x << 13;
    x ^= x >> 7;
    x ^= x << 17;
    *state = x;
    return (float)(x >> 40) / (float)(1ull << 24); /* mod.rs:687-689 */
}

/* sample_with_rng from step 3 on, sampling/mod.rs:487-564; softmax_candidates, mod.rs:617-638.  The candidate
 * values are the logits after steps 0-2 (bias, penalties, grammar), which leave this restatement's scope. */
uint32_t oxq_ref_sample_candidates(const float *vals, const uint32_t *idx, size_t k, float temperature,
                                   float min_p, float top_p, uint64_t *rng_state, float *probs_out,
                                   size_t *n_left_out) {
    if (probs_out) {
        for (size_t i = 0; i < k; i++) {
            probs_out[i] = 0.0f;
        }
    }
    if (n_left_out) {
        *n_left_out = k ? 1 : 0;
    }
    if (k == 0) {
        return 0;
    }
    /* step 3: greedy shortcut; the first candidate is argmax (largest value, lowest index) */
    if (temperature <= 0.0f || k == 1) {
        if (probs_out) {
            probs_out[0] = 1.0f;
        }
        return idx[0];
    }
    float *p = (float *)malloc(k * sizeof(float));
    uint32_t *ids = (uint32_t *)malloc(k * sizeof(uint32_t));
    memcpy(ids, idx, k * sizeof(uint32_t));
    /* step 4: every logit times 1 / temperature (the order of the candidates does not change) */
    if (temperature != 1.0f) {
        const float inv_temp = 1.0f / temperature;
        for (size_t i = 0; i < k; i++) {
            p[i] = vals[i] * inv_temp;
        }
    } else {
        for (size_t i = 0; i < k; i++) {
            p[i] = vals[i];
        }
    }
    /* step 7: softmax_candidates */
    float max_logit = -INFINITY;
    for (size_t i = 0; i < k; i++) {
        max_logit = fmaxf(max_logit, p[i]); /* f32::max: a NaN operand is ignored */
    }
    float sum = 0.0f;
    for (size_t i = 0; i < k; i++) {
        p[i] = expf(p[i] - max_logit);
        sum += p[i];
    }
    if (sum > 0.0f) {
        for (size_t i = 0; i < k; i++) {
            p[i] /= sum;
        }
    }
    size_t n = k;
    /* step 8: min-p, retain p >= min_p * p[0] (order kept) */
    if (min_p > 0.0f && n > 0) {
        const float threshold = min_p * p[0];
        size_t w = 0;
        for (size_t i = 0; i < n; i++) {
            if (p[i] >= threshold) {
                p[w] = p[i];
                ids[w] = ids[i];
                w++;
            }
        }
        n = w;
    }
    /* step 9: top-p */
    if (top_p < 1.0f && n > 0) {
        float cumulative = 0.0f;
        size_t cutoff = n;
        for (size_t i = 0; i < n; i++) {
            cumulative += p[i];
            if (cumulative >= top_p) {
                cutoff = i + 1;
                break;
            }
        }
        n = cutoff;
    }
    /* step 10: renormalise */
    float total = 0.0f;
    for (size_t i = 0; i < n; i++) {
        total += p[i];
    }
    if (total > 0.0f && total != 1.0f) {
        for (size_t i = 0; i < n; i++) {
            p[i] /= total;
        }
    }
    if (probs_out) {
        for (size_t i = 0; i < n; i++) {
            probs_out[i] = p[i];
        }
    }
    if (n_left_out) {
        *n_left_out = n;
    }
    /* step 11: the draw */
    uint32_t token;
    if (n == 0) {
        token = idx[0]; /* argmax of the processed logits */
    } else if (n == 1) {
        token = ids[0];
    } else {
        const float r = oxq_ref_xorshift64_next_f32(rng_state);
        float cumulative = 0.0f;
        token = ids[n - 1]; /* fallback: the last candidate */
        for (size_t i = 0; i < n; i++) {
            cumulative += p[i];
            if (r < cumulative) {
                token = ids[i];
                break;
            }
        }
    }
    free(p);
    free(ids);
    return token;
}

/* apply_logit_bias_and_banned_tokens, sampling/mod.rs:573-593; apply_repetition_penalty, mod.rs:596-613 */
void oxq_ref_logits_edit(float *logits, size_t n, const uint32_t *banned, size_t n_banned,
                         const uint32_t *bias_tokens, const float *bias_values, size_t n_bias,
                         const uint32_t *recent, size_t n_recent, size_t window, float repetition_penalty) {
    for (size_t i = 0; i < n_banned; i++) {
        if (banned[i] < n) {
            logits[banned[i]] = -INFINITY;
        }
    }
    for (size_t i = 0; i < n_bias; i++) {
        const size_t idx = bias_tokens[i];
        if (idx < n && isfinite(logits[idx])) {
            logits[idx] += bias_values[i];
        }
    }
    if (repetition_penalty == 1.0f || n_recent == 0) {
        return;
    }
    const size_t start = n_recent > window ? n_recent - window : 0; /* saturating_sub */
    for (size_t i = start; i < n_recent; i++) {
        const size_t idx = recent[i];
        if (idx < n) {
            if (logits[idx] > 0.0f) {
                logits[idx] /= repetition_penalty;
            } else {
                logits[idx] *= repetition_penalty;
            }
        }
    }
}
