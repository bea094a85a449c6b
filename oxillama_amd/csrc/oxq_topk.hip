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

__device__ __forceinline__ uint64_t topk_key(float v, uint32_t index) {
    uint32_t b = __builtin_bit_cast(uint32_t, v);
    b = (b & 0x80000000u) ? ~b : (b | 0x80000000u);  // unsigned order == float order
    if (v != v) b = 0;                                // NaN ranks below everything
    return ((uint64_t)b << 32) | (uint64_t)(0xFFFFFFFFu - index);
}
__device__ __forceinline__ float topk_value(uint64_t key) {
    uint32_t b = (uint32_t)(key >> 32);
    b = (b & 0x80000000u) ? (b & 0x7FFFFFFFu) : ~b;
    return __builtin_bit_cast(float, b);
}

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

uint32_t topk_items(size_t n) {  // elements per lane in stage 1 so that at most 256 slices (of 64 lanes) result
    const size_t per = (n + 16383) / 16384;
    return per <= 8 ? 8 : per <= 16 ? 16 : per <= 32 ? 32 : per <= 64 ? 64 : 0;
}

size_t topk_workspace_bytes(size_t n, size_t k) {
    const uint32_t items = topk_items(n);
    if (items == 0 || k == 0 || k > 256 || k > n) return 0;
    const size_t slices = (n + 64 * items - 1) / (64 * items);
    return slices * k * sizeof(uint64_t);
}

hipError_t launch_topk(const float *x, uint32_t n, uint32_t k, float *out_vals, uint32_t *out_idx, void *workspace,
                       hipStream_t stream) {
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

}  // namespace oxq
