// Mixture-of-experts layer around the grouped expert matmul, on the device (gfx950): what
// MoeFfn::forward of the reference (crates/oxillama-arch/src/common/moe.rs:184-258) does besides
// the experts' projections -- router logits, softmax, top-k selection and renormalised weights,
// the grouping of (token, expert) pairs by expert, the quantized activation rows in grouped
// order, and the weighted sum of the selected experts' outputs per token.
//
// Everything here is latency-bound bookkeeping over a few thousand elements, or elementwise
// fp32 traffic; the work is laid out so that the result does not depend on scheduling: no
// atomics, grouped rows in ascending (token, choice) order inside each expert.
#include "oxq_device.hpp"
#include "oxq_internal.hpp"
#include "oxq_q8_encode.hpp"

namespace oxq {

// One work group per token.  Wave w forms the logits of experts w, w+4, ... (lane-strided dot
// product, wave sum); lane 0 of wave 0 then runs the softmax and the selection serially in the
// reference's order (moe.rs:201-250): max, exp(l - max), sum in ascending expert order, divide;
// k times the largest remaining weight, the lower index on ties; weights divided by the sum of
// the selected ones (1/k when that sum is <= 1e-9).  n_exp floats of dynamic LDS.
__global__ __launch_bounds__(256) void moe_route_kernel(const float *__restrict__ router, const float *__restrict__ x,
                                                       int32_t *__restrict__ experts, float *__restrict__ weights,
                                                       uint32_t n_exp, uint32_t hidden, uint32_t k) {
    extern __shared__ float probs[];
    const uint32_t t = blockIdx.x, wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const float *xr = x + (size_t)t * hidden;
    for (uint32_t e = wave; e < n_exp; e += 4) {
        const float *rr = router + (size_t)e * hidden;
        float acc = 0.0f;
        for (uint32_t c = lane; c < hidden; c += 64) acc += rr[c] * xr[c];
        acc = wave_sum(acc);
        if (lane == 0) probs[e] = acc;
    }
    __syncthreads();
    if (threadIdx.x != 0) return;
    float max_logit = -INFINITY;
    for (uint32_t e = 0; e < n_exp; e++) max_logit = fmaxf(max_logit, probs[e]);
    float exp_sum = 0.0f;
    for (uint32_t e = 0; e < n_exp; e++) {
        const float v = expf(probs[e] - max_logit);
        probs[e] = v;
        exp_sum += v;
    }
    if (exp_sum > 0.0f) {
        for (uint32_t e = 0; e < n_exp; e++) probs[e] /= exp_sum;
    } else {
        const float uniform = 1.0f / (float)n_exp;
        for (uint32_t e = 0; e < n_exp; e++) probs[e] = uniform;
    }
    int32_t *sel = experts + (size_t)t * k;
    float *wt = weights + (size_t)t * k;
    float selected_sum = 0.0f;
    for (uint32_t r = 0; r < k; r++) {
        uint32_t best = 0;
        float best_v = -1.0f;  // weights are >= 0; taken entries are marked -2
        for (uint32_t e = 0; e < n_exp; e++) {
            const float v = probs[e];
            if (v > best_v) {
                best_v = v;
                best = e;
            }
        }
        // NaN weights (a NaN logit) never compare greater: fall back to the first untaken expert
        if (best_v < 0.0f) {
            for (uint32_t e = 0; e < n_exp; e++)
                if (probs[e] != -2.0f) {
                    best = e;
                    best_v = probs[e];
                    break;
                }
        }
        probs[best] = -2.0f;
        sel[r] = (int32_t)best;
        wt[r] = best_v;
        selected_sum += best_v;
    }
    for (uint32_t r = 0; r < k; r++) wt[r] = selected_sum > 1e-9f ? wt[r] / selected_sum : 1.0f / (float)k;
}

// One work group per expert e.  Pass 1 counts the pairs routed to experts below e (the first
// grouped row of e); pass 2 walks the pairs in ascending p = token * k + choice and gives the
// matching ones consecutive rows.  Writes offsets[e + 1] (and offsets[0]), pair_token[row] and
// token_rows[p]; no work group reads what another writes.
__global__ __launch_bounds__(256) void moe_group_kernel(const int32_t *__restrict__ experts, uint32_t n_pairs,
                                                       uint32_t k, int32_t *__restrict__ offsets,
                                                       int32_t *__restrict__ pair_token,
                                                       int32_t *__restrict__ token_rows) {
    __shared__ uint32_t wave_cnt[4];
    const int32_t e = (int32_t)blockIdx.x;
    const uint32_t wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    uint32_t below = 0;  // per wave, the same in every lane
    for (uint32_t p0 = 0; p0 < n_pairs; p0 += 256) {
        const uint32_t p = p0 + threadIdx.x;
        below += (uint32_t)__popcll(__ballot(p < n_pairs && experts[p] < e));
    }
    if (lane == 0) wave_cnt[wave] = below;
    __syncthreads();
    uint32_t run = wave_cnt[0] + wave_cnt[1] + wave_cnt[2] + wave_cnt[3];
    __syncthreads();
    for (uint32_t p0 = 0; p0 < n_pairs; p0 += 256) {
        const uint32_t p = p0 + threadIdx.x;
        const bool match = p < n_pairs && experts[p] == e;
        const unsigned long long ballot = __ballot(match);
        if (lane == 0) wave_cnt[wave] = (uint32_t)__popcll(ballot);
        __syncthreads();
        uint32_t before = 0, total = 0;
        for (uint32_t w = 0; w < 4; w++) {
            before += w < wave ? wave_cnt[w] : 0u;
            total += wave_cnt[w];
        }
        if (match) {
            const uint32_t row = run + before + (uint32_t)__popcll(ballot & ((1ull << lane) - 1ull));
            pair_token[row] = (int32_t)(p / k);
            token_rows[p] = (int32_t)row;
        }
        run += total;
        __syncthreads();
    }
    if (threadIdx.x == 0) {
        offsets[e + 1] = (int32_t)run;
        if (e == 0) offsets[0] = 0;
    }
}

// Row r of the grouped activation matrix = the Q8_0 blocks of token pair_token[r]'s input vector
// (every selected expert runs on the same input, moe.rs:246).  Eight lanes per block as in the quantizer.
__global__ __launch_bounds__(256) void moe_gather_quantize_kernel(const float *__restrict__ x,
                                                                 const int32_t *__restrict__ pair_token,
                                                                 uint8_t *__restrict__ out, size_t n_blocks,
                                                                 uint32_t blocks_per_row, uint32_t hidden) {
    const size_t t = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const size_t blk = t >> 3;
    const uint32_t j = (uint32_t)(t & 7);
    const bool valid = blk < n_blocks;
    float v[4] = {0.0f, 0.0f, 0.0f, 0.0f};
    if (valid) {
        const size_t row = blk / blocks_per_row, b = blk % blocks_per_row;
        load4(v, x + (size_t)pair_token[row] * hidden + b * 32 + 4 * j);
    }
    encode_q8_0_lanes(v, valid, out + blk * 34, j);
}

// out[t][c] = sum over the token's selected experts, in selection order, of weight * expert_out
// (moe.rs:236-254: output zeroed, then `*o += weight * e` per expert; multiply and add rounded separately).
__global__ __launch_bounds__(256) void moe_combine_kernel(const float *__restrict__ y_pairs,
                                                         const int32_t *__restrict__ token_rows,
                                                         const float *__restrict__ weights, float *__restrict__ out,
                                                         uint32_t n_tokens, uint32_t top_k, uint32_t hidden) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= (size_t)n_tokens * hidden) return;
    const uint32_t t = (uint32_t)(i / hidden), c = (uint32_t)(i % hidden);
    float o = 0.0f;
    for (uint32_t j = 0; j < top_k; j++) {
        const float e = y_pairs[(size_t)token_rows[t * top_k + j] * hidden + c];
        const float p = weights[t * top_k + j] * e;
        o += p;
    }
    out[i] = o;
}

hipError_t launch_moe_gather_quantize(const float *x, const int32_t *pair_token, uint8_t *out, size_t n_pairs,
                                      uint32_t hidden, hipStream_t stream) {
    const uint32_t bpr = hidden / 32;
    const size_t n_blocks = n_pairs * bpr;
    if (n_blocks == 0) return hipSuccess;
    hipLaunchKernelGGL(moe_gather_quantize_kernel, dim3((unsigned)((n_blocks * 8 + 255) / 256)), dim3(256), 0, stream, x,
                       pair_token, out, n_blocks, bpr, hidden);
    return hipGetLastError();
}

hipError_t launch_moe_combine(const float *y_pairs, const int32_t *token_rows, const float *weights, float *out,
                              uint32_t n_tokens, uint32_t top_k, uint32_t hidden, hipStream_t stream) {
    const size_t n = (size_t)n_tokens * hidden;
    if (n == 0) return hipSuccess;
    hipLaunchKernelGGL(moe_combine_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, stream, y_pairs, token_rows,
                       weights, out, n_tokens, top_k, hidden);
    return hipGetLastError();
}

hipError_t launch_moe_route(const float *router, const float *x, int32_t *experts, float *weights, uint32_t n_tokens,
                            uint32_t n_exp, uint32_t hidden, uint32_t k, int32_t *offsets, int32_t *pair_token,
                            int32_t *token_rows, hipStream_t stream) {
    if (n_tokens == 0 || n_exp == 0) return hipSuccess;
    hipLaunchKernelGGL(moe_route_kernel, dim3(n_tokens), dim3(256), n_exp * sizeof(float), stream, router, x, experts,
                       weights, n_exp, hidden, k);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return e;
    hipLaunchKernelGGL(moe_group_kernel, dim3(n_exp), dim3(256), 0, stream, experts, n_tokens * k, k, offsets,
                       pair_token, token_rows);
    return hipGetLastError();
}

}  // namespace oxq
