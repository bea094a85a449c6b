// Exact top-k of an fp32 vector on the device (gfx950): the candidate list the reference's sampler
// builds from the logits -- (index, value) pairs sorted by value, largest first, cut to top_k
// (crates/oxillama-runtime/src/sampling/mod.rs:500-509) -- and, for k = 1, its argmax (first of
// equal maxima, mod.rs:652-662).  The reference's sort leaves the order of exactly equal values
// open; here the lower index comes first.  Index work: results are exact.
//
// Values become 64-bit keys (order-preserving bits of the float, then the complement of the
// index), so one unsigned maximum decides value and tie at once.  Stage 1: every wave selects the
// k largest keys of its slice (held in registers) by k rounds of a wave maximum (DPP, no LDS, no
// barrier).  Stage 2: one wave merges the slices' sorted lists by their heads (four lists per lane).
#include "oxq_device.hpp"
#include "oxq_internal.hpp"

namespace oxq {

// Slice s = elements [s * 64 * ITEMS, (s + 1) * 64 * ITEMS), one wave each: its k largest keys, largest
// first, to cand[s * k .. s * k + k); slots beyond the slice's size hold key 0.  Waves work on their own.
template <int ITEMS>
__global__ __launch_bounds__(256) void topk_slices_kernel(const float *__restrict__ x, uint32_t n, uint32_t k,
                                                         uint32_t n_slices, uint64_t *__restrict__ cand) {
    const uint32_t lane = threadIdx.x & 63;
    const uint32_t slice = __builtin_amdgcn_readfirstlane(blockIdx.x * 4 + (threadIdx.x >> 6));
    if (slice >= n_slices) return;
    const uint32_t base = slice * 64 * ITEMS;
    uint64_t key[ITEMS];
#pragma unroll
    for (int j = 0; j < ITEMS; j++) {
        const uint32_t i = base + j * 64 + lane;
        key[j] = i < n ? topk_key(x[i], i) : 0;
    }
    for (uint32_t r = 0; r < k; r++) {
        uint64_t m = key[0];
#pragma unroll
        for (int j = 1; j < ITEMS; j++) m = max_u64(m, key[j]);
        const uint64_t best = wave_max_u64(m);
#pragma unroll
        for (int j = 0; j < ITEMS; j++)
            if (key[j] == best) key[j] = 0;  // keys are unique (they carry the index); 0 == 0 is harmless
        if (lane == 0) cand[(size_t)slice * k + r] = best;
    }
}

// Merge of n_lists (<= 256) descending lists of k keys by one wave: lane l walks lists l, l + 64, l + 128, l + 192.
__global__ __launch_bounds__(64) void topk_merge_kernel(const uint64_t *__restrict__ cand, uint32_t n_lists, uint32_t k,
                                                       float *__restrict__ out_vals, uint32_t *__restrict__ out_idx) {
    const uint32_t lane = threadIdx.x;
    uint32_t head[4] = {0, 0, 0, 0};
    uint64_t cur[4];
#pragma unroll
    for (int j = 0; j < 4; j++) cur[j] = lane + 64 * j < n_lists ? cand[(size_t)(lane + 64 * j) * k] : 0;
    for (uint32_t r = 0; r < k; r++) {
        const uint64_t best = wave_max_u64(max_u64(max_u64(cur[0], cur[1]), max_u64(cur[2], cur[3])));
#pragma unroll
        for (int j = 0; j < 4; j++)
            if (cur[j] == best && best != 0) {  // one lane, one list: its next key (a dependent load per round)
                head[j]++;
                cur[j] = head[j] < k ? cand[(size_t)(lane + 64 * j) * k + head[j]] : 0;
            }
        if (lane == 0) {
            out_vals[r] = topk_value(best);
            out_idx[r] = 0xFFFFFFFFu - (uint32_t)best;
        }
    }
}

// ---- larger k: one work group, a filter by group maxima, then a radix select in LDS -----------------------
// 1. Every thread takes the maximum of its share of the keys (no atomics).  The k-th largest of these 1024
//    maxima, T1, is a lower bound of the k-th largest key overall: k different threads each hold a key >= T1.
// 2. A second pass copies every key >= T1 to LDS.  For logits that is barely more than k keys (k = 256 of
//    128256: about 300); at most SEL_CAP fit.
// 3. The k-th largest of the survivors, T, is found digit by digit from the top (8-bit digits: histogram of the
//    digit over the keys that match the digits found so far, suffix scan from the top bin; the bin in which the
//    count crosses what is still wanted is T's next digit), until the keys at or above the prefix are exactly k.
//    They are ranked among themselves by counting and written in order.
// If step 2 overflows (the large values all sit in a few threads' shares, which takes an adversarial layout) the
// same digit search runs over the keys in memory with 12-bit digits instead: exact as well, several passes slower.
// Keys are unique (they carry the index), so every count is exact and ties come out lower index first, as in
// the two-stage kernels above.
constexpr uint32_t SEL_CAP = 8192, SEL_THREADS = 1024;

// Suffix scan over the bins from the top: the digit d with count(bins > d) < want <= count(bins >= d), and
// those two counts.  All threads call; nb <= 4 * SEL_THREADS bins; result broadcast through `res`.
template <uint32_t THREADS = SEL_THREADS>
__device__ __forceinline__ void select_digit(const uint32_t *hist, uint32_t nb, uint32_t want, uint32_t *wave_tot,
                                             uint32_t *res, uint32_t &digit, uint32_t &above, uint32_t &equal) {
    const uint32_t tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    uint32_t p = 0;
    if (4 * tid < nb) p = hist[4 * tid] + hist[4 * tid + 1] + hist[4 * tid + 2] + hist[4 * tid + 3];
    uint32_t v = p;  // sum over the lanes at or above this one
    for (uint32_t off = 1; off < 64; off <<= 1) {
        const uint32_t y = __shfl_down(v, off, 64);
        if (lane + off < 64) v += y;
    }
    if (lane == 0) wave_tot[wave] = v;
    __syncthreads();
    uint32_t higher = 0;
    for (uint32_t w = wave + 1; w < THREADS / 64; w++) higher += wave_tot[w];
    const uint32_t incl = v + higher, excl = incl - p;
    if (excl < want && incl >= want) {  // exactly one thread: the crossing is inside its four bins
        uint32_t run = excl;
        for (int b = 3; b >= 0; b--) {
            const uint32_t c = hist[4 * tid + b];
            if (run + c >= want) {
                res[0] = 4 * tid + b;
                res[1] = run;
                res[2] = c;
                break;
            }
            run += c;
        }
    }
    __syncthreads();
    digit = res[0];
    above = res[1];
    equal = res[2];
    __syncthreads();  // res and wave_tot may be rewritten by the next call
}

// One count for the bin of `d`; lanes of a wave that share the first active lane's bin go in as one addition
// (same-address LDS atomics serialise, and masked logits put tens of thousands of -inf into one bin).
__device__ __forceinline__ void hist_add(uint32_t *hist, uint32_t d, bool valid) {
    const uint64_t active = __ballot(valid);
    if (active == 0) return;
    const uint32_t leader = (uint32_t)__builtin_ctzll(active);
    const uint32_t d0 = (uint32_t)__builtin_amdgcn_readlane((int)d, (int)leader);
    const uint64_t same = __ballot(valid && d == d0);
    if (__builtin_popcountll(same) >= 8) {
        if ((threadIdx.x & 63) == leader) atomicAdd(&hist[d0], (uint32_t)__builtin_popcountll(same));
        if (valid && d != d0) atomicAdd(&hist[d], 1u);
    } else if (valid) {
        atomicAdd(&hist[d], 1u);
    }
}

struct SelectShared {
    uint32_t hist[4096];
    uint32_t wave_tot[SEL_THREADS / 64], res[3], counter;
};

// The smallest threshold t (low bits zero) such that exactly `want` of the keys `each` visits are >= t, found
// W bits at a time from the top.  `each(fn)` calls fn(key, valid) for every key, the same number of times in every
// thread of a wave; all threads of the work group call this function.
template <int W, uint32_t THREADS = SEL_THREADS, class Each>
__device__ __forceinline__ uint64_t kth_threshold(Each &&each, uint32_t want, SelectShared &sh) {
    static_assert((1u << W) <= 4 * THREADS, "a thread sums four bins in the scan");
    const uint32_t tid = threadIdx.x;
    uint64_t prefix = 0;  // the digits found so far
    uint32_t done = 0;    // how many bits that is
    while (true) {
        const uint32_t w = min((uint32_t)W, 64u - done), nb = 1u << w;
        for (uint32_t b = tid; b < (nb < 4 ? 4 : nb); b += THREADS) sh.hist[b] = 0;
        __syncthreads();
        const uint32_t shift = 64 - done - w;
        each([&](uint64_t key, bool valid) {
            const bool match = valid && (done == 0 || (key >> (64 - done)) == prefix);
            hist_add(sh.hist, (uint32_t)(key >> shift) & (nb - 1), match);
        });
        __syncthreads();
        uint32_t digit, above, equal;
        select_digit<THREADS>(sh.hist, nb, want, sh.wave_tot, sh.res, digit, above, equal);
        prefix = (prefix << w) | digit;
        done += w;
        want -= above;  // the threshold is the want-th largest of the keys that match the prefix
        if (equal == want || done == 64) return done == 64 ? prefix : prefix << (64 - done);
    }
}

__global__ __launch_bounds__(SEL_THREADS) void topk_select_kernel(const float *__restrict__ x, uint32_t n, uint32_t k,
                                                                 float *__restrict__ out_vals,
                                                                 uint32_t *__restrict__ out_idx) {
    __shared__ SelectShared sh;
    __shared__ uint64_t cand[SEL_CAP];
    __shared__ uint64_t sel[256];
    const uint32_t tid = threadIdx.x;
    const bool vec4 = (reinterpret_cast<uintptr_t>(x) & 15) == 0;
    // every key of the vector: 16-byte loads, four in flight per thread (16 keys per thread and trip), when the
    // vector starts on a 16-byte boundary
    auto each_in_memory = [&](auto &&fn) {
        if (vec4) {
            for (uint32_t i0 = 0; i0 < n; i0 += 16 * SEL_THREADS) {
                u32x4 v[4];
                uint32_t idx[4];
#pragma unroll
                for (int u = 0; u < 4; u++) {
                    idx[u] = i0 + 4 * (u * SEL_THREADS + tid);
                    v[u] = idx[u] + 4 <= n ? *reinterpret_cast<const u32x4 *>(x + idx[u]) : u32x4{0, 0, 0, 0};
                }
#pragma unroll
                for (int u = 0; u < 4; u++)
#pragma unroll
                    for (int e = 0; e < 4; e++) {
                        const uint32_t bits = v[u][e];
                        fn(topk_key(__builtin_bit_cast(float, bits), idx[u] + e), idx[u] + 4 <= n);
                    }
            }
            if ((n & 3u) && tid < 64) {  // the last n % 4 keys, by the first wave
                const uint32_t i = (n & ~3u) + tid;
                fn(i < n ? topk_key(x[i], i) : 0, i < n);
            }
            return;
        }
        for (uint32_t i0 = 0; i0 < n; i0 += 4 * SEL_THREADS) {
            float v[4];
            uint32_t idx[4];
#pragma unroll
            for (int u = 0; u < 4; u++) {
                idx[u] = i0 + u * SEL_THREADS + tid;
                v[u] = idx[u] < n ? x[idx[u]] : 0.0f;
            }
#pragma unroll
            for (int u = 0; u < 4; u++) fn(topk_key(v[u], idx[u]), idx[u] < n);
        }
    };
    uint32_t n_cand = 0;
    auto each_in_lds = [&](auto &&fn) {
        for (uint32_t j0 = 0; j0 < n_cand; j0 += SEL_THREADS) {
            const uint32_t j = j0 + tid;
            fn(j < n_cand ? cand[j] : 0, j < n_cand);
        }
    };
    // 1. the k-th largest of the threads' maxima
    uint64_t best = 0;
    each_in_memory([&](uint64_t key, bool valid) { best = valid ? max_u64(best, key) : best; });
    cand[tid] = best;  // a thread without keys holds 0, which is below every key
    n_cand = SEL_THREADS;
    __syncthreads();
    const uint64_t t1 = kth_threshold<8>(each_in_lds, k, sh);
    // 2. the keys at or above it, to LDS
    if (tid == 0) sh.counter = 0;
    __syncthreads();
    each_in_memory([&](uint64_t key, bool valid) {
        if (valid && key >= t1) {
            const uint32_t pos = atomicAdd(&sh.counter, 1u);
            if (pos < SEL_CAP) cand[pos] = key;
        }
    });
    __syncthreads();
    n_cand = sh.counter;
    __syncthreads();
    // 3. the k-th largest key
    uint64_t t;
    if (n_cand <= SEL_CAP) {
        t = kth_threshold<8>(each_in_lds, k, sh);
    } else {
        t = kth_threshold<12>(each_in_memory, k, sh);
        if (tid == 0) sh.counter = 0;
        __syncthreads();
        each_in_memory([&](uint64_t key, bool valid) {
            if (valid && key >= t) cand[atomicAdd(&sh.counter, 1u)] = key;  // exactly k of them
        });
        __syncthreads();
        n_cand = sh.counter;
        __syncthreads();
    }
    // the k keys, then each one's rank among them
    if (tid == 0) sh.counter = 0;
    __syncthreads();
    for (uint32_t j = tid; j < n_cand; j += SEL_THREADS) {
        const uint64_t key = cand[j];
        if (key >= t) sel[atomicAdd(&sh.counter, 1u)] = key;
    }
    __syncthreads();
    if (tid < k) {
        const uint64_t mine = sel[tid];
        uint32_t rank = 0;
        for (uint32_t j = 0; j < k; j++) rank += sel[j] > mine ? 1u : 0u;
        out_vals[rank] = topk_value(mine);
        out_idx[rank] = 0xFFFFFFFFu - (uint32_t)mine;
    }
}

// ---- the same selection spread over the chip: two launches -------------------------------------------------------
// One work group reading 128256 logits twice is what the kernel above spends its time on (31-39 us).  Here the vector
// is cut into G slices; a work group per slice keeps its slice's keys in LDS and selects the slice's k largest with
// the same digit search (a slice with at most k keys passes them all on); the G * k survivors (<= SEL_CAP) go to the
// workspace, and one work group selects and ranks the k largest of those.  Exact for the same reason: every key of
// the overall top k is among its own slice's top k.  12-bit digits: two rounds settle 24 bits of the value, which
// separates a few thousand logits (8-bit digits take three; measured 14.6 us against 19.1 for k = 40 in a replayed
// graph, 23.9 against 27.8 for k = 256).  After the lm_head GEMV (71 us): 87 us for the pair with k = 40.
constexpr uint32_t SPREAD_THREADS = 1024;  // (four waves instead of sixteen measured slower: the key loops get longer)
__global__ __launch_bounds__(SPREAD_THREADS) void topk_slice_select_kernel(const float *__restrict__ x, uint32_t n, uint32_t k,
                                                                       uint32_t slice_len, uint64_t *__restrict__ ws) {
    __shared__ SelectShared sh;
    __shared__ uint64_t cand[SEL_CAP];
    const uint32_t tid = threadIdx.x;
    const uint32_t lo = blockIdx.x * slice_len, hi = min(n, lo + slice_len);
    const uint32_t n_cand = hi > lo ? hi - lo : 0;
    for (uint32_t j = tid; j < n_cand; j += SPREAD_THREADS) cand[j] = topk_key(x[lo + j], lo + j);
    if (tid == 0) sh.counter = 0;
    __syncthreads();
    auto each_in_lds = [&](auto &&fn) {
        for (uint32_t j0 = 0; j0 < n_cand; j0 += SPREAD_THREADS) {
            const uint32_t j = j0 + tid;
            fn(j < n_cand ? cand[j] : 0, j < n_cand);
        }
    };
    uint64_t *out = ws + (size_t)blockIdx.x * k;
    if (n_cand <= k) {  // the whole slice, padded with keys that rank below everything
        for (uint32_t j = tid; j < k; j += SPREAD_THREADS) out[j] = j < n_cand ? cand[j] : 0;
        return;
    }
    const uint64_t t = kth_threshold<12, SPREAD_THREADS>(each_in_lds, k, sh);
    for (uint32_t j = tid; j < n_cand; j += SPREAD_THREADS) {
        const uint64_t key = cand[j];
        if (key >= t) out[atomicAdd(&sh.counter, 1u)] = key;  // exactly k of them
    }
}

// The k largest of n_cand (<= SEL_CAP) keys, ranked, to the outputs.
__global__ __launch_bounds__(SPREAD_THREADS) void topk_final_kernel(const uint64_t *__restrict__ ws, uint32_t n_cand, uint32_t k,
                                                                float *__restrict__ out_vals, uint32_t *__restrict__ out_idx) {
    __shared__ SelectShared sh;
    __shared__ uint64_t cand[SEL_CAP];
    __shared__ uint64_t sel[256];
    const uint32_t tid = threadIdx.x;
    for (uint32_t j = tid; j < n_cand; j += SPREAD_THREADS) cand[j] = ws[j];
    if (tid == 0) sh.counter = 0;
    __syncthreads();
    auto each_in_lds = [&](auto &&fn) {
        for (uint32_t j0 = 0; j0 < n_cand; j0 += SPREAD_THREADS) {
            const uint32_t j = j0 + tid;
            fn(j < n_cand ? cand[j] : 0, j < n_cand);
        }
    };
    const uint64_t t = kth_threshold<12, SPREAD_THREADS>(each_in_lds, k, sh);
    for (uint32_t j = tid; j < n_cand; j += SPREAD_THREADS) {
        const uint64_t key = cand[j];
        if (key >= t) sel[atomicAdd(&sh.counter, 1u)] = key;
    }
    __syncthreads();
    if (tid < k) {
        const uint64_t mine = sel[tid];
        uint32_t rank = 0;
        for (uint32_t j = 0; j < k; j++) rank += sel[j] > mine ? 1u : 0u;
        out_vals[rank] = topk_value(mine);
        out_idx[rank] = 0xFFFFFFFFu - (uint32_t)mine;
    }
}

// Slices of the two-launch form for (n, k): 0 if it does not apply (every slice must fit the LDS key buffer, and the
// slices' survivors together as well).
static uint32_t topk_spread_slices(size_t n, size_t k) {
    if (k == 0 || k > 256 || n <= 4096 || n > 0xFFFFFFFFull) return 0;  // a short vector: one work group does it
    uint32_t g = (uint32_t)(SEL_CAP / k);
    if (g > 64) g = 64;  // 16 to 128 slices measured alike (128256 logits: 17-19 us with 8-bit digits); 64 is the flat middle
    const size_t len = (n + g - 1) / g;
    return len <= SEL_CAP ? g : 0;
}

uint32_t topk_items(size_t n) {  // elements per lane in stage 1 so that at most 256 slices (of 64 lanes) result
    const size_t per = (n + 16383) / 16384;
    return per <= 8 ? 8 : per <= 16 ? 16 : per <= 32 ? 32 : per <= 64 ? 64 : 0;
}

// From this k on the radix select is the faster of the two one-work-group forms (128256 logits: 31-39 us whatever k, against 13 us at
// k = 8, 26 us at 32, 36 us at 48, 47 us at 64, 173 us at 256 for the two-stage kernels).
constexpr uint32_t TOPK_SELECT_MIN_K = 40;
// ... and from this k on, for vectors of more than 4096 values whose slices fit, the two-launch form is faster still.
constexpr uint32_t TOPK_SPREAD_MIN_K = 16;

size_t topk_workspace_bytes(size_t n, size_t k) {
    const uint32_t items = topk_items(n);
    if (items == 0 || k == 0 || k > 256 || k > n) return 0;
    const size_t slices = (n + 64 * items - 1) / (64 * items);
    const size_t spread = (size_t)topk_spread_slices(n, k) * k * sizeof(uint64_t);
    const size_t waves = slices * k * sizeof(uint64_t);
    return spread > waves ? spread : waves;
}

hipError_t launch_topk(const float *x, uint32_t n, uint32_t k, float *out_vals, uint32_t *out_idx, void *workspace,
                       hipStream_t stream) {
    if (k >= TOPK_SPREAD_MIN_K) {
        if (const uint32_t g = topk_spread_slices(n, k)) {  // slices selected side by side, then their survivors
            const uint32_t len = (n + g - 1) / g;
            uint64_t *ws = static_cast<uint64_t *>(workspace);
            hipLaunchKernelGGL(topk_slice_select_kernel, dim3(g), dim3(SPREAD_THREADS), 0, stream, x, n, k, len, ws);
            hipError_t e = hipGetLastError();
            if (e != hipSuccess) return e;
            hipLaunchKernelGGL(topk_final_kernel, dim3(1), dim3(SPREAD_THREADS), 0, stream, ws, g * k, k, out_vals, out_idx);
            return hipGetLastError();
        }
    }
    if (k >= TOPK_SELECT_MIN_K) {  // radix select by one work group; needs no workspace
        hipLaunchKernelGGL(topk_select_kernel, dim3(1), dim3(SEL_THREADS), 0, stream, x, n, k, out_vals, out_idx);
        return hipGetLastError();
    }
    const uint32_t items = topk_items(n);
    const uint32_t slices = (n + 64 * items - 1) / (64 * items);
    const dim3 grid((slices + 3) / 4);
    uint64_t *cand = static_cast<uint64_t *>(workspace);
    switch (items) {
    case 8: hipLaunchKernelGGL(topk_slices_kernel<8>, grid, dim3(256), 0, stream, x, n, k, slices, cand); break;
    case 16: hipLaunchKernelGGL(topk_slices_kernel<16>, grid, dim3(256), 0, stream, x, n, k, slices, cand); break;
    case 32: hipLaunchKernelGGL(topk_slices_kernel<32>, grid, dim3(256), 0, stream, x, n, k, slices, cand); break;
    case 64: hipLaunchKernelGGL(topk_slices_kernel<64>, grid, dim3(256), 0, stream, x, n, k, slices, cand); break;
    default: return hipErrorInvalidValue;
    }
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return e;
    hipLaunchKernelGGL(topk_merge_kernel, dim3(1), dim3(64), 0, stream, cand, slices, k, out_vals, out_idx);
    return hipGetLastError();
}

// The sampler from its candidate list on: sample_with_rng's steps 3 to 11 (crates/oxillama-runtime/src/sampling/
// mod.rs:487-564; softmax_candidates :617-638; Xorshift64 :669-690) on the k <= 256 candidates that the top-k above
// leaves, largest logit first -- so that a token id, not a candidate list, leaves the device.  One work group.  What
// the reference does element by element is done by all threads (the scaling, the exponentials, the divisions), what
// it does as a running sum in candidate order (softmax sum, top-p, renormalisation, the draw) by thread 0 in that
// order, so that every fp32 value is the reference's: exp is the C library's (expf_libm), the divisions are
// correctly rounded.  rng_state is advanced only when more than one candidate survives, as in the reference.
__global__ __launch_bounds__(256) void sample_candidates_kernel(const float *__restrict__ vals, const uint32_t *__restrict__ idx,
                                                                uint32_t k, float temperature, float min_p, float top_p,
                                                                uint64_t *__restrict__ rng_state, uint32_t *__restrict__ token_out,
                                                                float *__restrict__ probs_out) {
    __shared__ float p[256];
    __shared__ uint32_t ids[256];
    __shared__ float s_val;
    __shared__ uint32_t s_n;
    const uint32_t t = threadIdx.x;
    if (temperature <= 0.0f || k == 1) {  // step 3: greedy; the first candidate is the argmax
        if (t == 0) *token_out = idx[0];
        if (probs_out && t < k) probs_out[t] = t == 0 ? 1.0f : 0.0f;
        return;
    }
    if (t < k) {
        float v = vals[t];
        if (temperature != 1.0f) v = v * (1.0f / temperature);  // step 4
        p[t] = v;
        ids[t] = idx[t];
    }
    __syncthreads();
    if (t == 0) {  // step 7: the maximum (f32::max: a NaN operand is ignored)
        float m = -INFINITY;
        for (uint32_t i = 0; i < k; i++) m = fmaxf(m, p[i]);
        s_val = m;
    }
    __syncthreads();
    const float max_logit = s_val;
    if (t < k) p[t] = expf_libm(p[t] - max_logit);
    __syncthreads();
    if (t == 0) {
        float sum = 0.0f;
        for (uint32_t i = 0; i < k; i++) sum += p[i];
        s_val = sum;
    }
    __syncthreads();
    const float sum = s_val;
    if (t < k && sum > 0.0f) p[t] = p[t] / sum;
    __syncthreads();
    if (t == 0) {
        uint32_t n = k;
        if (min_p > 0.0f) {  // step 8
            const float threshold = min_p * p[0];
            uint32_t w = 0;
            for (uint32_t i = 0; i < n; i++)
                if (p[i] >= threshold) {
                    p[w] = p[i];
                    ids[w] = ids[i];
                    w++;
                }
            n = w;
        }
        if (top_p < 1.0f && n > 0) {  // step 9
            float cumulative = 0.0f;
            uint32_t cutoff = n;
            for (uint32_t i = 0; i < n; i++) {
                cumulative += p[i];
                if (cumulative >= top_p) {
                    cutoff = i + 1;
                    break;
                }
            }
            n = cutoff;
        }
        float total = 0.0f;  // step 10
        for (uint32_t i = 0; i < n; i++) total += p[i];
        s_val = total;
        s_n = n;
    }
    __syncthreads();
    const uint32_t n = s_n;
    const float total = s_val;
    if (t < n && total > 0.0f && total != 1.0f) p[t] = p[t] / total;
    __syncthreads();
    if (probs_out && t < k) probs_out[t] = t < n ? p[t] : 0.0f;
    if (t == 0) {  // step 11
        uint32_t token;
        if (n == 0) {
            token = idx[0];
        } else if (n == 1) {
            token = ids[0];
        } else {
            uint64_t x = *rng_state;
            x ^= x << 13;
            x ^= x >> 7;
            x ^= x << 17;
            *rng_state = x;
            const float r = (float)(x >> 40) / 16777216.0f;
            float cumulative = 0.0f;
            token = ids[n - 1];
            for (uint32_t i = 0; i < n; i++) {
                cumulative += p[i];
                if (r < cumulative) {
                    token = ids[i];
                    break;
                }
            }
        }
        *token_out = token;
    }
}

// Steps 0 and 1 of sample_with_rng on the logits in place (sampling/mod.rs:573-613): banned tokens to -inf, the
// bias added where the logit is still finite (each biased token once: the reference's map), then the repetition
// penalty over the last `window` recent tokens.  One work group; the three steps are ordered by barriers (they may
// touch the same logit).  The reference applies the penalty once per OCCURRENCE of a token, in order: here the lane
// that holds a token's first occurrence in the window applies it as many times as the token occurs, to the value
// in a register -- the same operations on the same value in the same order.
__global__ __launch_bounds__(256) void logits_edit_kernel(float *__restrict__ logits, uint32_t n,
                                                          const uint32_t *__restrict__ banned, uint32_t n_banned,
                                                          const uint32_t *__restrict__ bias_tokens,
                                                          const float *__restrict__ bias_values, uint32_t n_bias,
                                                          const uint32_t *__restrict__ recent, uint32_t n_window,
                                                          float penalty) {
    const uint32_t t = threadIdx.x;
    for (uint32_t i = t; i < n_banned; i += 256)
        if (banned[i] < n) logits[banned[i]] = -INFINITY;
    __threadfence_block();
    __syncthreads();
    for (uint32_t i = t; i < n_bias; i += 256) {
        const uint32_t idx = bias_tokens[i];
        if (idx < n) {
            const float v = logits[idx];
            if (__builtin_isfinite(v)) logits[idx] = v + bias_values[i];
        }
    }
    __threadfence_block();
    __syncthreads();
    if (penalty == 1.0f || n_window == 0) return;
    for (uint32_t i = t; i < n_window; i += 256) {
        const uint32_t tok = recent[i];
        if (tok >= n) continue;
        uint32_t count = 0;
        bool first = true;
        for (uint32_t j = 0; j < n_window; j++) {
            const bool same = recent[j] == tok;
            count += same ? 1u : 0u;
            first = first && !(same && j < i);
        }
        if (!first) continue;
        float v = logits[tok];
        for (uint32_t c = 0; c < count; c++) v = v > 0.0f ? v / penalty : v * penalty;
        logits[tok] = v;
    }
}

hipError_t launch_logits_edit(float *logits, uint32_t n, const uint32_t *banned, uint32_t n_banned, const uint32_t *bias_tokens,
                              const float *bias_values, uint32_t n_bias, const uint32_t *recent, uint32_t n_window,
                              float penalty, hipStream_t stream) {
    hipLaunchKernelGGL(logits_edit_kernel, dim3(1), dim3(256), 0, stream, logits, n, banned, n_banned, bias_tokens,
                       bias_values, n_bias, recent, n_window, penalty);
    return hipGetLastError();
}

hipError_t launch_sample_candidates(const float *vals, const uint32_t *idx, uint32_t k, float temperature, float min_p,
                                    float top_p, uint64_t *rng_state, uint32_t *token_out, float *probs_out,
                                    hipStream_t stream) {
    hipLaunchKernelGGL(sample_candidates_kernel, dim3(1), dim3(256), 0, stream, vals, idx, k, temperature, min_p, top_p,
                       rng_state, token_out, probs_out);
    return hipGetLastError();
}

}  // namespace oxq
