/*
 * oxq_oracle.h -- TEST INFRASTRUCTURE, NOT PRODUCT CODE.
 *
 * Scalar C restatement of oxillama-quant's CPU kernels for the quantized-matmul
 * path (reference = /root/reference/crates/oxillama-quant/src, abbreviated Q/).
 * Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may load
 * this library; the shipped HIP path never calls it.
 *
 * Every function names the reference lines whose operation order it follows.
 * Build with -O2 -ffp-contract=off -fno-fast-math: Rust neither contracts
 * a*b+c into an fma nor reassociates floating point.
 *
 * Pinning (what each group of functions is checked against, see tests/):
 *   f16 <-> f32            all 65 536 halves and random floats vs F16C hardware
 *   quantizers             closed-form invariants and the reference's own test
 *                          vectors (Q/quantize.rs:225-445)
 *   dequant_block, gemv    the reference's hand-built block tests
 *                          (Q/reference/{q4_0,q8_0,q4_k,q6_k,iq4_xs}.rs tests)
 *   matvec_q8_fused        fused == unfused identities, accumulate semantics,
 *                          zero cases, AVX2-tier fixtures (Q/simd/avx2/ tests)
 *   block integer sums     brute force from dequantized integer weights
 *   IQ4_XS fused           the reference has no working implementation (the
 *                          trait default indexes a 32-entry scratch with 256
 *                          weights, Q/traits.rs:135,158-166); the integer form
 *                          defined here is pinned against the reference gemv
 *                          applied to dequantized activations.
 */
#ifndef OXQ_ORACLE_H
#define OXQ_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* GgufTensorType ids, crates/oxillama-gguf/src/types.rs:72-150 */
enum {
    OXQ_REF_Q4_0 = 2,
    OXQ_REF_Q8_0 = 8,
    OXQ_REF_Q4_K = 12,
    OXQ_REF_Q6_K = 14,
    OXQ_REF_IQ4_XS = 23,
    /* restated in oxq_oracle_more.c */
    OXQ_REF_Q4_1 = 3,
    OXQ_REF_Q5_0 = 6,
    OXQ_REF_Q5_1 = 7,
    OXQ_REF_Q8_1 = 9,
    OXQ_REF_Q2_K = 10,
    OXQ_REF_Q3_K = 11,
    OXQ_REF_Q5_K = 13,
    OXQ_REF_IQ4_NL = 20
};

/* QuantError variants, Q/error.rs:10-71 */
enum {
    OXQ_REF_OK = 0,
    OXQ_REF_UNSUPPORTED_TYPE = 1,
    OXQ_REF_BLOCK_SIZE_MISMATCH = 2,
    OXQ_REF_DIMENSION_MISMATCH = 3, /* a = expected, b = got */
    OXQ_REF_KERNEL_ERROR = 4,
    OXQ_REF_BLOCK_COUNT_MISMATCH = 5,
    OXQ_REF_BUFFER_TOO_SMALL = 6, /* a = needed, b = available */
    OXQ_REF_INTERNAL = 7
};

/* matvec_q8_fused tiers */
enum {
    OXQ_REF_TIER_SCALAR = 0,     /* what the *Ref kernels run */
    OXQ_REF_TIER_AVX2 = 1,       /* operation order of Q/simd/avx2 fused rows */
    OXQ_REF_TIER_Q4_0_STANDALONE = 2 /* Q/reference/q4_0.rs:159 */
};

typedef struct {
    int code;
    size_t a;
    size_t b;
} oxq_ref_status;

size_t oxq_ref_block_size(uint32_t type);
size_t oxq_ref_block_bytes(uint32_t type);

uint16_t oxq_ref_f32_to_f16(float v);
float oxq_ref_f16_to_f32(uint16_t h);

oxq_ref_status oxq_ref_quantize_f32_to_q8_0(const float *x, size_t n, uint8_t *out);
oxq_ref_status oxq_ref_quantize_f32_to_q4_0(const float *x, size_t n, uint8_t *out);

oxq_ref_status oxq_ref_dequant_block(uint32_t type, const uint8_t *block, size_t block_len,
                                     float *out, size_t out_len);

oxq_ref_status oxq_ref_gemv(uint32_t type, const uint8_t *w, size_t w_len, size_t n_rows,
                            size_t n_cols, const float *x, size_t x_len, float *y, size_t y_len);

oxq_ref_status oxq_ref_gemm(uint32_t type, const uint8_t *w, size_t w_len, const float *x,
                            float *y, size_t m, size_t n, size_t k);

oxq_ref_status oxq_ref_matvec_q8_fused(uint32_t type, int tier, const uint8_t *w, size_t w_len,
                                       const uint8_t *acts, size_t acts_len, float *out,
                                       size_t out_len, size_t n_rows, size_t n_cols);

/* Integer-dot form shared by every format: per (row, integer group) the exact
 * int32 sum, then one fp32 term per group.  Group = 32 weights (one Q8_0
 * activation block) for Q4_0/Q8_0/Q4_K/IQ4_XS and 16 weights for Q6_K. */
oxq_ref_status oxq_ref_matvec_q8_intdot(uint32_t type, const uint8_t *w, size_t w_len,
                                        const uint8_t *acts, size_t acts_len, float *out,
                                        size_t out_len, size_t n_rows, size_t n_cols);

/* sums[row * groups_per_row + g]; groups_per_row = n_cols/32 (n_cols/16 for Q6_K).
 * Q4_0: sum (q-8)*a; Q8_0: sum w*a; Q4_K: sum q*a (unsigned nibble); Q6_K:
 * sum (q-32)*a; IQ4_XS: sum kvalues[q]*a.  n_cols must be a block multiple. */
oxq_ref_status oxq_ref_block_sums(uint32_t type, const uint8_t *w, size_t w_len,
                                  const uint8_t *acts, size_t acts_len, int32_t *sums,
                                  size_t n_rows, size_t n_cols);

/* Prefill: quantize each of the m activation rows to Q8_0, then m fused matvecs
 * into a zeroed y[m x n] (gemm semantics of Q/reference/q4_k.rs:186-201 applied
 * to the Q8_0-activation path). */
oxq_ref_status oxq_ref_gemm_q8(uint32_t type, int tier, const uint8_t *w, size_t w_len,
                               const float *x, float *y, size_t m, size_t n, size_t k);

/* Multi-threaded row split of the AVX2-order fused matvec: parallel_gemv
 * semantics (Q/parallel.rs:70-77), used only for the CPU baseline timing. */
oxq_ref_status oxq_ref_matvec_q8_fused_mt(uint32_t type, int tier, const uint8_t *w, size_t w_len,
                                          const uint8_t *acts, size_t acts_len, float *out,
                                          size_t out_len, size_t n_rows, size_t n_cols,
                                          int n_threads);

/* ---- the callers' glue (oxq_oracle_linear.c) ---- */

/* swiglu_inplace, crates/oxillama-arch/src/common/swiglu.rs:15-21 */
void oxq_ref_swiglu_inplace(float *gate, const float *up, size_t n);
/* RmsNorm::forward_to, crates/oxillama-arch/src/common/rms_norm.rs:49-66 */
void oxq_ref_rmsnorm_forward_to(const float *input, const float *weight, float eps, size_t n,
                                float *output);
/* LoraAdapter::new / apply, crates/oxillama-quant/src/lora.rs:43-124 */
oxq_ref_status oxq_ref_lora_new(size_t a_len, size_t b_len, size_t rank, size_t in_features,
                                size_t out_features);
oxq_ref_status oxq_ref_lora_apply(const float *a, const float *b, size_t rank, float scale,
                                  size_t in_features, size_t out_features, const float *input,
                                  size_t input_len, float *output, size_t output_len);
/* QuantLinear::forward, crates/oxillama-arch/src/common/linear.rs:77-98, gemv on the
 * Q8_0-activation path; bias / lora_a / lora_b may be NULL. */
oxq_ref_status oxq_ref_linear_forward(uint32_t type, int tier, const uint8_t *w, size_t w_len,
                                      size_t n_rows, size_t n_cols, const float *bias, size_t bias_len,
                                      const float *lora_a, const float *lora_b, size_t rank, float scale,
                                      const float *input, size_t input_len, float *output,
                                      size_t output_len);

/* argmax and the truncated, sorted candidate list of the sampler,
 * crates/oxillama-runtime/src/sampling/mod.rs:500-509,652-662 */
uint32_t oxq_ref_argmax(const float *values, size_t n);
void oxq_ref_topk(const float *values, size_t n, size_t k, float *out_vals, uint32_t *out_idx);
/* Steps 0 and 1 of sample_with_rng on the logits, in place: apply_logit_bias_and_banned_tokens (sampling/mod.rs:
 * 573-593: banned tokens to -inf, then bias added where the logit is still finite) and apply_repetition_penalty
 * (mod.rs:596-613: for every token of the last `window` entries of recent, in order and once per occurrence, a
 * positive logit is divided by the penalty, any other multiplied; nothing for penalty == 1).  Token ids past n are
 * skipped.  bias_tokens holds each token once (the reference's map). */
void oxq_ref_logits_edit(float *logits, size_t n, const uint32_t *banned, size_t n_banned,
                         const uint32_t *bias_tokens, const float *bias_values, size_t n_bias,
                         const uint32_t *recent, size_t n_recent, size_t window, float repetition_penalty);
/* Xorshift64::new / next_u64 / next_f32, sampling/mod.rs:669-690: the sampler's generator.  *state is
 * advanced; a zero seed is replaced as new() does. */
uint64_t oxq_ref_xorshift64_seed(uint64_t seed);
float oxq_ref_xorshift64_next_f32(uint64_t *state);
/* The tail of sample_with_rng, sampling/mod.rs:487-564, on the k candidates that steps 5 and 6 (sort, truncate to
 * top_k) leave, largest logit first: greedy shortcut (temperature <= 0 or k == 1), temperature scaling, softmax
 * over the candidates, min-p, top-p, renormalisation, and the draw against one rng.next_f32() -- which is taken
 * only when more than one candidate is left, as in the reference.  probs_out (optional, k floats) receives the
 * final probabilities, zeros past the survivors; n_left_out (optional) their count.  Returns the token id. */
uint32_t oxq_ref_sample_candidates(const float *vals, const uint32_t *idx, size_t k, float temperature,
                                   float min_p, float top_p, uint64_t *rng_state, float *probs_out,
                                   size_t *n_left_out);

/* ---- mixture-of-experts feed-forward (oxq_oracle_moe.c), crates/oxillama-arch/src/common/moe.rs ---- */

/* Expert::forward, moe.rs:75-127 (dense fp32) */
oxq_ref_status oxq_ref_expert_forward(const float *gate, size_t gate_len, const float *up, size_t up_len,
                                      const float *down, size_t down_len, size_t hidden, size_t inter,
                                      const float *input, float *output);
/* routing of MoeFfn::forward, moe.rs:189-250; outputs hold min(top_k, n_exp) entries */
oxq_ref_status oxq_ref_moe_route(const float *router, size_t router_len, size_t n_exp, size_t hidden,
                                 size_t top_k, const float *input, uint32_t *experts_out, float *weights_out,
                                 size_t *k_out);
/* output[i] += weight * expert_out[i], moe.rs:254-256 */
void oxq_ref_moe_accumulate(float *output, const float *expert_out, float weight, size_t n);
/* MoeFfn::forward, moe.rs:184-258, dense experts stored back to back */
oxq_ref_status oxq_ref_moe_forward(const float *router, size_t router_len, const float *gate_all,
                                   const float *up_all, const float *down_all, size_t n_exp, size_t hidden,
                                   size_t inter, size_t top_k, const float *input, float *output);
/* the same with the experts' projections in a block format, through matvec_q8_fused */
oxq_ref_status oxq_ref_expert_forward_q(uint32_t type, int tier, const uint8_t *gate, const uint8_t *up,
                                        const uint8_t *down, size_t hidden, size_t inter,
                                        const uint8_t *input_q8, float *output);
oxq_ref_status oxq_ref_moe_forward_q(uint32_t type, int tier, const float *router, size_t router_len,
                                     const uint8_t *gate_all, const uint8_t *up_all, const uint8_t *down_all,
                                     size_t n_exp, size_t hidden, size_t inter, size_t top_k, const float *input,
                                     float *output, uint32_t *sel_out, float *wt_out);

#ifdef __cplusplus
}
#endif
#endif
