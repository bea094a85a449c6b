/*
 * oxq_oracle_moe.c -- TEST INFRASTRUCTURE, NOT PRODUCT CODE.
 *
 * Scalar C restatement of the reference's mixture-of-experts feed-forward layer
 * (/root/reference/crates/oxillama-arch/src/common/moe.rs): Expert::forward and
 * MoeFfn::forward on dense fp32 weights, and the same layer with the experts' three
 * projections held in a GGUF block format and run through the Q8_0-activation fused
 * matvec, which is what the grouped expert matmul on the device computes.  Same rules as
 * oxq_oracle.c: reference operation order, -ffp-contract=off -fno-fast-math.
 *
 * Pinning (tests/test_oracle_moe.py):
 *   expert_forward    the reference's tests (moe.rs:275-320): all-ones expert against its
 *                     closed form n*h*h/(1+exp(-h)), zero input, wrong gate size; float64
 *                     recomputation on random weights
 *   moe_route         the reference's cases (moe.rs:323-405): one-hot router, uniform router
 *                     (weights 1/k), top_k above the expert count, top_k = 0; invariants
 *                     (weights sum to 1, descending, softmax closed form in float64)
 *   moe_forward       identical experts make the output independent of routing; float64
 *                     recomputation of the weighted sum on random experts
 *   moe_forward_q     equals moe_forward when weights and activations are exactly
 *                     representable in the block format (Q8_0 experts with integer weights)
 */
#include <math.h>
#include <stdlib.h>
#include <string.h>

#include "oxq_oracle.h"

static oxq_ref_status st(int code, size_t a, size_t b) {
    oxq_ref_status s = {code, a, b};
    return s;
}

/* row . input with the reference's iterator sum: ascending index, from 0.0 */
static float dot_seq(const float *row, const float *x, size_t n) {
    float s = 0.0f;
    for (size_t i = 0; i < n; i++) {
        s += row[i] * x[i];
    }
    return s;
}

/* Expert::forward, moe.rs:75-127.  A wrong buffer length is ArchError::InvalidShape (moe.rs:33-58),
 * reported here as DIMENSION_MISMATCH {expected, got}. */
oxq_ref_status oxq_ref_expert_forward(const float *gate, size_t gate_len, const float *up, size_t up_len,
                                      const float *down, size_t down_len, size_t hidden, size_t inter,
                                      const float *input, float *output) {
    if (gate_len != inter * hidden) {
        return st(OXQ_REF_DIMENSION_MISMATCH, inter * hidden, gate_len);
    }
    if (up_len != inter * hidden) {
        return st(OXQ_REF_DIMENSION_MISMATCH, inter * hidden, up_len);
    }
    if (down_len != hidden * inter) {
        return st(OXQ_REF_DIMENSION_MISMATCH, hidden * inter, down_len);
    }
    float *gate_vec = (float *)calloc(inter ? inter : 1, sizeof(float));
    float *up_vec = (float *)calloc(inter ? inter : 1, sizeof(float));
    for (size_t i = 0; i < inter; i++) {
        gate_vec[i] = dot_seq(gate + i * hidden, input, hidden); /* :83-90 */
    }
    for (size_t i = 0; i < inter; i++) {
        float sigmoid = 1.0f / (1.0f + expf(-gate_vec[i])); /* :94 */
        gate_vec[i] *= sigmoid;                             /* :95 */
    }
    for (size_t i = 0; i < inter; i++) {
        up_vec[i] = dot_seq(up + i * hidden, input, hidden); /* :99-106 */
    }
    for (size_t i = 0; i < inter; i++) {
        up_vec[i] *= gate_vec[i]; /* :110-112 */
    }
    for (size_t i = 0; i < hidden; i++) {
        output[i] = dot_seq(down + i * inter, up_vec, inter); /* :115-122 */
    }
    free(gate_vec);
    free(up_vec);
    return st(OXQ_REF_OK, 0, 0);
}

/* Steps 1-4 of MoeFfn::forward, moe.rs:189-240: router logits, stable softmax, the top-k experts
 * by descending weight, weights renormalised over the selected ones.  The reference's
 * sort_unstable_by leaves the order of equal weights open; this restatement takes the lower
 * index first.  experts_out / weights_out hold min(top_k, n_exp) entries, *k_out that count. */
oxq_ref_status oxq_ref_moe_route(const float *router, size_t router_len, size_t n_exp, size_t hidden,
                                 size_t top_k, const float *input, uint32_t *experts_out, float *weights_out,
                                 size_t *k_out) {
    if (router_len != n_exp * hidden) { /* :153-160 */
        return st(OXQ_REF_DIMENSION_MISMATCH, n_exp * hidden, router_len);
    }
    if (top_k == 0) { /* :168-172, ArchError::InvalidConfig */
        return st(OXQ_REF_KERNEL_ERROR, 1, 0);
    }
    float *p = (float *)calloc(n_exp ? n_exp : 1, sizeof(float));
    unsigned char *taken = (unsigned char *)calloc(n_exp ? n_exp : 1, 1);
    for (size_t i = 0; i < n_exp; i++) {
        p[i] = dot_seq(router + i * hidden, input, hidden); /* :191-199 */
    }
    float max_logit = -INFINITY;
    for (size_t i = 0; i < n_exp; i++) {
        max_logit = fmaxf(max_logit, p[i]); /* :202-205 */
    }
    float exp_sum = 0.0f;
    for (size_t i = 0; i < n_exp; i++) {
        p[i] = expf(p[i] - max_logit); /* :206-209 */
    }
    for (size_t i = 0; i < n_exp; i++) {
        exp_sum += p[i]; /* :210 */
    }
    if (exp_sum > 0.0f) {
        for (size_t i = 0; i < n_exp; i++) {
            p[i] /= exp_sum; /* :212-215 */
        }
    } else {
        float uniform = 1.0f / (float)n_exp; /* :217-220 */
        for (size_t i = 0; i < n_exp; i++) {
            p[i] = uniform;
        }
    }
    size_t k = top_k < n_exp ? top_k : n_exp; /* :233 */
    for (size_t r = 0; r < k; r++) {          /* :224-234 */
        size_t best = n_exp;
        for (size_t i = 0; i < n_exp; i++) {
            if (!taken[i] && (best == n_exp || p[i] > p[best])) {
                best = i;
            }
        }
        taken[best] = 1;
        experts_out[r] = (uint32_t)best;
    }
    float selected_sum = 0.0f;
    for (size_t r = 0; r < k; r++) {
        selected_sum += p[experts_out[r]]; /* :237 */
    }
    for (size_t r = 0; r < k; r++) { /* :246-250 */
        weights_out[r] = selected_sum > 1e-9f ? p[experts_out[r]] / selected_sum : 1.0f / (float)k;
    }
    *k_out = k;
    free(p);
    free(taken);
    return st(OXQ_REF_OK, 0, 0);
}

/* `*o += weight * e`, moe.rs:254-256 */
void oxq_ref_moe_accumulate(float *output, const float *expert_out, float weight, size_t n) {
    for (size_t i = 0; i < n; i++) {
        output[i] += weight * expert_out[i];
    }
}

/* MoeFfn::forward, moe.rs:184-258, experts dense: expert e's gate / up at gate_all / up_all +
 * e * inter * hidden, its down at down_all + e * hidden * inter. */
oxq_ref_status oxq_ref_moe_forward(const float *router, size_t router_len, const float *gate_all,
                                   const float *up_all, const float *down_all, size_t n_exp, size_t hidden,
                                   size_t inter, size_t top_k, const float *input, float *output) {
    uint32_t *sel = (uint32_t *)calloc(n_exp ? n_exp : 1, sizeof(uint32_t));
    float *wt = (float *)calloc(n_exp ? n_exp : 1, sizeof(float));
    float *expert_out = (float *)calloc(hidden ? hidden : 1, sizeof(float));
    size_t k = 0;
    oxq_ref_status s = oxq_ref_moe_route(router, router_len, n_exp, hidden, top_k, input, sel, wt, &k);
    if (s.code == OXQ_REF_OK) {
        memset(output, 0, hidden * sizeof(float)); /* :240-242 */
        for (size_t r = 0; r < k && s.code == OXQ_REF_OK; r++) {
            size_t e = sel[r], mat = inter * hidden;
            s = oxq_ref_expert_forward(gate_all + e * mat, mat, up_all + e * mat, mat, down_all + e * mat, mat,
                                       hidden, inter, input, expert_out); /* :252 */
            if (s.code == OXQ_REF_OK) {
                oxq_ref_moe_accumulate(output, expert_out, wt[r], hidden);
            }
        }
    }
    free(sel);
    free(wt);
    free(expert_out);
    return s;
}

/* One expert with its projections in block format `type`: the input's Q8_0 blocks against the
 * gate and up rows (matvec_q8_fused), swiglu_inplace, the product quantized to Q8_0, the down
 * rows -- the dense feed-forward of the quantized models with an expert's matrices. */
oxq_ref_status oxq_ref_expert_forward_q(uint32_t type, int tier, const uint8_t *gate, const uint8_t *up,
                                        const uint8_t *down, size_t hidden, size_t inter,
                                        const uint8_t *input_q8, float *output) {
    size_t bs = oxq_ref_block_size(type), bb = oxq_ref_block_bytes(type);
    if (bs == 0) {
        return st(OXQ_REF_UNSUPPORTED_TYPE, type, 0);
    }
    if (hidden % bs || inter % bs) {
        return st(OXQ_REF_DIMENSION_MISMATCH, bs, hidden % bs ? hidden : inter);
    }
    size_t gu_bytes = inter * (hidden / bs) * bb, down_bytes = hidden * (inter / bs) * bb;
    size_t in_q8 = hidden / 32 * 34, h_q8 = inter / 32 * 34;
    float *g = (float *)calloc(inter ? inter : 1, sizeof(float));
    float *u = (float *)calloc(inter ? inter : 1, sizeof(float));
    uint8_t *hq = (uint8_t *)calloc(h_q8 ? h_q8 : 1, 1);
    oxq_ref_status s = oxq_ref_matvec_q8_fused(type, tier, gate, gu_bytes, input_q8, in_q8, g, inter, inter, hidden);
    if (s.code == OXQ_REF_OK) {
        s = oxq_ref_matvec_q8_fused(type, tier, up, gu_bytes, input_q8, in_q8, u, inter, inter, hidden);
    }
    if (s.code == OXQ_REF_OK) {
        oxq_ref_swiglu_inplace(g, u, inter);
        s = oxq_ref_quantize_f32_to_q8_0(g, inter, hq);
    }
    if (s.code == OXQ_REF_OK) {
        memset(output, 0, hidden * sizeof(float));
        s = oxq_ref_matvec_q8_fused(type, tier, down, down_bytes, hq, h_q8, output, hidden, hidden, inter);
    }
    free(g);
    free(u);
    free(hq);
    return s;
}

/* MoeFfn::forward with quantized experts; the router stays fp32 as in the reference.  sel_out /
 * wt_out (optional) receive the routing decision. */
oxq_ref_status oxq_ref_moe_forward_q(uint32_t type, int tier, const float *router, size_t router_len,
                                     const uint8_t *gate_all, const uint8_t *up_all, const uint8_t *down_all,
                                     size_t n_exp, size_t hidden, size_t inter, size_t top_k, const float *input,
                                     float *output, uint32_t *sel_out, float *wt_out) {
    size_t bs = oxq_ref_block_size(type), bb = oxq_ref_block_bytes(type);
    if (bs == 0) {
        return st(OXQ_REF_UNSUPPORTED_TYPE, type, 0);
    }
    if (hidden % bs || inter % bs) {
        return st(OXQ_REF_DIMENSION_MISMATCH, bs, hidden % bs ? hidden : inter);
    }
    uint32_t *sel = (uint32_t *)calloc(n_exp ? n_exp : 1, sizeof(uint32_t));
    float *wt = (float *)calloc(n_exp ? n_exp : 1, sizeof(float));
    float *expert_out = (float *)calloc(hidden ? hidden : 1, sizeof(float));
    uint8_t *xq = (uint8_t *)calloc(hidden / 32 * 34 + 1, 1);
    size_t k = 0;
    oxq_ref_status s = oxq_ref_moe_route(router, router_len, n_exp, hidden, top_k, input, sel, wt, &k);
    if (s.code == OXQ_REF_OK) {
        s = oxq_ref_quantize_f32_to_q8_0(input, hidden, xq);
    }
    if (s.code == OXQ_REF_OK) {
        size_t gu_bytes = inter * (hidden / bs) * bb, down_bytes = hidden * (inter / bs) * bb;
        memset(output, 0, hidden * sizeof(float));
        for (size_t r = 0; r < k && s.code == OXQ_REF_OK; r++) {
            size_t e = sel[r];
            s = oxq_ref_expert_forward_q(type, tier, gate_all + e * gu_bytes, up_all + e * gu_bytes,
                                         down_all + e * down_bytes, hidden, inter, xq, expert_out);
            if (s.code == OXQ_REF_OK) {
                oxq_ref_moe_accumulate(output, expert_out, wt[r], hidden);
            }
            if (sel_out) {
                sel_out[r] = sel[r];
            }
            if (wt_out) {
                wt_out[r] = wt[r];
            }
        }
    }
    free(sel);
    free(wt);
    free(expert_out);
    free(xq);
    return s;
}
