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

// One work group per token.  The 256 lanes form the logits together (16-byte loads, lane, wave and
// work-group sums); wave 0 then runs the softmax and the selection (moe.rs:201-250): max,
// exp(l - max), sum, divide; k rounds of "largest remaining weight, lower index on ties" as one
// 64-bit wave maximum over keys (weight bits, complemented index); weights divided by the sum of
// the selected ones in selection order (1/k when that sum is <= 1e-9).  Lane l owns experts l,
// l + 64, ... in LDS.  5 * n_exp floats of dynamic LDS.
//
// ONE (a launch for a single token, k <= n_exp): the work group goes on to what the grouping and
// the gather kernels would do for that token -- the k chosen experts in ascending order are the
// grouped rows (offsets[e] = how many chosen experts lie below e), every row belongs to token 0,
// and each row's activations are the token's Q8_0 blocks, written k times while the logits are
// formed.  Same tables and bytes as the separate launches.
// The logits of experts e0 .. e0 + 7 for one token, by the 256 threads of a work group: per-thread sums over the
// columns (16-byte loads), lane sums, one partial per wave into part[4 * q + wave].
constexpr int ROUTE_EP = 8;  // experts per pass: their loads are in flight together
template <bool ONE>
__device__ __forceinline__ void route_logits_pass(const float *__restrict__ router, const float *__restrict__ xr, uint32_t e0,
                                                  uint32_t n_exp, uint32_t hidden, uint32_t k, uint8_t *__restrict__ acts,
                                                  float *part) {
    constexpr int EP = ROUTE_EP;
    const uint32_t wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const uint32_t n4 = (hidden & 3) == 0 ? hidden / 4 : 0;
    const float *rr[EP];
    float acc[EP];
    for (int q = 0; q < EP; q++) {
        rr[q] = router + (size_t)min(e0 + q, n_exp - 1) * hidden;
        acc[q] = 0.0f;
    }
    if (n4) {
        for (uint32_t c = threadIdx.x; c < n4; c += 256) {
            float xv[4], rv[EP][4];
            load4(xv, xr + 4 * c);
#pragma unroll
            for (int q = 0; q < EP; q++) load4(rv[q], rr[q] + 4 * c);
#pragma unroll
            for (int q = 0; q < EP; q++)
                for (int i = 0; i < 4; i++) acc[q] += rv[q][i] * xv[i];
            if (ONE && e0 == 0) {
                // the activation rows are k copies of the token's Q8_0 blocks whichever experts get chosen:
                // written from the values in hand (eight consecutive lanes hold one block, as in the quantizer;
                // hidden is a multiple of 32 here, so a block's lanes are in the loop together)
                for (uint32_t r = 0; r < k; r++)
                    encode_q8_0_lanes(xv, true, acts + ((size_t)r * (hidden / 32) + c / 8) * 34, c & 7);
            }
        }
    } else {
        for (uint32_t c = threadIdx.x; c < hidden; c += 256)
            for (int q = 0; q < EP; q++) acc[q] += rr[q][c] * xr[c];
    }
#pragma unroll
    for (int q = 0; q < EP; q++) {
        const float v = wave_sum(acc[q]);
        if (lane == 0 && e0 + q < n_exp) part[4 * q + wave] = v;
    }
}

// Many experts: the logits by a launch of their own, a work group per (token, eight experts) -- the same sums in the
// same order as inside moe_route_kernel, which then starts from them.  (One work group per token walks 128 experts of
// 2048 columns in 35 us.)
template <bool ONE>
__global__ __launch_bounds__(256) void moe_logits_kernel(const float *__restrict__ router, const float *__restrict__ x,
                                                        float *__restrict__ logits, uint32_t n_exp, uint32_t hidden,
                                                        uint32_t k, uint8_t *__restrict__ acts) {
    __shared__ float part[4 * ROUTE_EP];
    const uint32_t t = blockIdx.x, e0 = blockIdx.y * ROUTE_EP;
    route_logits_pass<ONE>(router, x + (size_t)t * hidden, e0, n_exp, hidden, k, acts, part);
    __syncthreads();
    if (threadIdx.x < ROUTE_EP && e0 + threadIdx.x < n_exp) {
        const uint32_t q = threadIdx.x;
        logits[(size_t)t * n_exp + e0 + q] = (part[4 * q] + part[4 * q + 1]) + (part[4 * q + 2] + part[4 * q + 3]);
    }
}

template <bool ONE>
__global__ __launch_bounds__(256) void moe_route_kernel(const float *__restrict__ router, const float *__restrict__ x,
                                                       int32_t *__restrict__ experts, float *__restrict__ weights,
                                                       uint32_t n_exp, uint32_t hidden, uint32_t k,
                                                       int32_t *__restrict__ offsets, int32_t *__restrict__ pair_token,
                                                       int32_t *__restrict__ token_rows, uint8_t *__restrict__ acts,
                                                       const float *__restrict__ logits) {
    extern __shared__ float lds[];
    float *probs = lds, *part = lds + n_exp;
    const uint32_t t = blockIdx.x, wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    if (logits) {  // formed by moe_logits_kernel
        for (uint32_t e = threadIdx.x; e < n_exp; e += 256) probs[e] = logits[(size_t)t * n_exp + e];
    } else {
        const float *xr = x + (size_t)t * hidden;
        for (uint32_t e0 = 0; e0 < n_exp; e0 += ROUTE_EP) route_logits_pass<ONE>(router, xr, e0, n_exp, hidden, k, acts, part + 4 * e0);
        __syncthreads();
        for (uint32_t e = threadIdx.x; e < n_exp; e += 256)
            probs[e] = (part[4 * e] + part[4 * e + 1]) + (part[4 * e + 2] + part[4 * e + 3]);
    }

    __syncthreads();
    int32_t *chosen = reinterpret_cast<int32_t *>(part);  // ONE: the selection, for the other waves (part is free now)

    if (wave == 0) {
        float m = -INFINITY;
        for (uint32_t e = lane; e < n_exp; e += 64) m = fmaxf(m, probs[e]);
        m = fmaxf(m, dpp_f<0xB1>(m));
        m = fmaxf(m, dpp_f<0x4E>(m));
        m = fmaxf(m, dpp_f<0x124>(m));
        m = fmaxf(m, dpp_f<0x128>(m));
        const float max_logit =
            fmaxf(fmaxf(readlane_f(m, 0), readlane_f(m, 16)), fmaxf(readlane_f(m, 32), readlane_f(m, 48)));
        float s = 0.0f;
        for (uint32_t e = lane; e < n_exp; e += 64) {
            const float v = expf_libm(probs[e] - max_logit);
            probs[e] = v;
            s += v;
        }
        const float exp_sum = wave_sum(s);
        const float uniform = 1.0f / (float)n_exp;
        for (uint32_t e = lane; e < n_exp; e += 64) probs[e] = exp_sum > 0.0f ? probs[e] / exp_sum : uniform;

        int32_t *sel = experts + (size_t)t * k;
        float *wt = weights + (size_t)t * k;
        float selected_sum = 0.0f;
        for (uint32_t r = 0; r < k; r++) {
            uint64_t best = 0;
            for (uint32_t e = lane; e < n_exp; e += 64) {
                const float v = probs[e];  // >= 0 (or NaN, which ranks first and is taken once); taken entries are -1
                const uint64_t key =
                    v < 0.0f ? 0 : ((uint64_t)__builtin_bit_cast(uint32_t, v) << 32) | (0xFFFFFFFFu - e);
                best = max_u64(best, key);
            }
            best = wave_max_u64(best);
            const uint32_t e = 0xFFFFFFFFu - (uint32_t)best;
            const float v = __builtin_bit_cast(float, (uint32_t)(best >> 32));
            if ((e & 63) == lane) probs[e] = -1.0f;  // the owner lane is the only one that reads it again
            selected_sum += v;
            if (lane == 0) {
                sel[r] = (int32_t)e;
                wt[r] = v;
                if (ONE) chosen[r] = (int32_t)e;
            }
        }
        if (lane == 0)
            for (uint32_t r = 0; r < k; r++) wt[r] = selected_sum > 1e-9f ? wt[r] / selected_sum : 1.0f / (float)k;
    }
    if (!ONE) return;

    __syncthreads();
    for (uint32_t e = threadIdx.x; e <= n_exp; e += 256) {
        int32_t below = 0;
        for (uint32_t r = 0; r < k; r++) below += chosen[r] < (int32_t)e ? 1 : 0;
        offsets[e] = below;
    }
    for (uint32_t p = threadIdx.x; p < k; p += 256) {
        int32_t row = 0;
        for (uint32_t r = 0; r < k; r++) row += chosen[r] < chosen[p] ? 1 : 0;
        token_rows[p] = row;
        pair_token[row] = 0;
    }
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
// splits > 1: an expert output is the sum, in index order, of `splits` partial results split_stride floats apart
// (the down matmul left its halves of k unadded).
__global__ __launch_bounds__(256) void moe_combine_kernel(const float *__restrict__ y_pairs,
                                                         const int32_t *__restrict__ token_rows,
                                                         const float *__restrict__ weights, float *__restrict__ out,
                                                         uint32_t n_tokens, uint32_t top_k, uint32_t hidden,
                                                         uint32_t splits, size_t split_stride) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= (size_t)n_tokens * hidden) return;
    const uint32_t t = (uint32_t)(i / hidden), c = (uint32_t)(i % hidden);
    float o = 0.0f;
    for (uint32_t j = 0; j < top_k; j++) {
        const size_t at = (size_t)token_rows[t * top_k + j] * hidden + c;
        float e = y_pairs[at];
        for (uint32_t s = 1; s < splits; s++) e += y_pairs[at + s * split_stride];
        const float p = weights[t * top_k + j] * e;
        o += p;
    }
    out[i] = o;
}

__global__ __launch_bounds__(256) void fill_zero_kernel(float *__restrict__ out, size_t n) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) out[i] = 0.0f;
}

// A fill by a kernel, not a memset node: callers may be capturing the stream into a graph.
hipError_t launch_fill_zero(float *out, size_t n, hipStream_t stream) {
    if (n == 0) return hipSuccess;
    hipLaunchKernelGGL(fill_zero_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, stream, out, n);
    return hipGetLastError();
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
                              uint32_t n_tokens, uint32_t top_k, uint32_t hidden, hipStream_t stream, uint32_t splits,
                              size_t split_stride) {
    const size_t n = (size_t)n_tokens * hidden;
    if (n == 0) return hipSuccess;
    hipLaunchKernelGGL(moe_combine_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, stream, y_pairs, token_rows,
                       weights, out, n_tokens, top_k, hidden, splits, split_stride);
    return hipGetLastError();
}

hipError_t launch_moe_route(const float *router, const float *x, int32_t *experts, float *weights, uint32_t n_tokens,
                            uint32_t n_exp, uint32_t hidden, uint32_t k, int32_t *offsets, int32_t *pair_token,
                            int32_t *token_rows, hipStream_t stream, uint8_t *acts_one, float *logits_scratch) {
    if (n_tokens == 0 || n_exp == 0) return hipSuccess;
    const size_t lds = 5 * n_exp * sizeof(float);
    // From 32 experts on (four passes of a token's work group and more), where the caller has room for n_tokens x n_exp
    // floats: the logits by a launch of their own.
    const float *logits = nullptr;
    if (logits_scratch && n_exp >= 32 && n_tokens <= 65535) {
        const dim3 grid(n_tokens, (n_exp + ROUTE_EP - 1) / ROUTE_EP);
        if (acts_one)
            hipLaunchKernelGGL(moe_logits_kernel<true>, grid, dim3(256), 0, stream, router, x, logits_scratch, n_exp, hidden, k,
                               acts_one);
        else
            hipLaunchKernelGGL(moe_logits_kernel<false>, grid, dim3(256), 0, stream, router, x, logits_scratch, n_exp, hidden, k,
                               acts_one);
        hipError_t e = hipGetLastError();
        if (e != hipSuccess) return e;
        logits = logits_scratch;
    }
    if (acts_one) {  // the caller checked: one token, a handful of choices, whole blocks
        hipLaunchKernelGGL(moe_route_kernel<true>, dim3(1), dim3(256), lds, stream, router, x, experts, weights, n_exp,
                           hidden, k, offsets, pair_token, token_rows, acts_one, logits);
        return hipGetLastError();
    }
    hipLaunchKernelGGL(moe_route_kernel<false>, dim3(n_tokens), dim3(256), lds, stream, router, x, experts, weights,
                       n_exp, hidden, k, offsets, pair_token, token_rows, acts_one, logits);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return e;
    hipLaunchKernelGGL(moe_group_kernel, dim3(n_exp), dim3(256), 0, stream, experts, n_tokens * k, k, offsets,
                       pair_token, token_rows);
    return hipGetLastError();
}

}  // namespace oxq
