// The vocabulary projection together with a short candidate list (greedy decoding, small top_k), in ONE launch:
//   logits = W[n_vocab x hidden] . x_q8   (the lm_head's fused matvec, crates/oxillama-quant/src/reference/q6_k.rs:212-354
//                                          for the usual Q6_K matrix)
//   the k <= 8 largest logits, largest first, with their token ids (crates/oxillama-runtime/src/sampling/mod.rs:500-509;
//   k = 1: the argmax, mod.rs:652-662)
// The GEMV is gemv_q8_cached's one-wave-per-row loop (oxq_gemv_kernel.hpp: same loads, same sums, same launch width --
// the logits are its logits bit for bit).  What is added sits after the last row batch, and uses no barrier but one:
//  * every wave has kept the logits of its row batches as 64-bit keys (value bits, then the complement of the index) in
//    registers, batch i in lane i; k rounds of a wave maximum (DPP) give the wave's k largest, in order;
//  * the first wave of the work group does the same over the four waves' lists and writes the work group's list to the
//    workspace -- every key of the overall top k is among its own work group's top k;
//  * a ticket counts the work groups that have done so (the lists are stored and read past the L2s); the one that
//    draws the last ticket reads all lists into LDS and merges them by their heads (a list per lane and turn), k rounds.
//    No work group waits for another: every wave exits after its own work.
// Tickets are library-owned words of device memory that every launch leaves at zero; a call takes the next of 1024 in
// turn, so calls that overlap on different streams do not share one.
// Measured on the 128256 x 4096 Q6_K matrix (GEMV alone 70.6 us): k = 1 / 4 / 8 74.7 / 77.5 / 81 us against 78.2 / 80.4 /
// 82.7 for the GEMV launch followed by the top-k launches.  Longer lists (top_k = 40) stay with those launches:
// selecting 40 of a work group's 500 logits and then 40 of 10200 by the last work group (digit search in LDS, 256
// threads) took 7 + 40 us behind the GEMV, against 15 us for the two top-k launches.
#include <algorithm>
#include <atomic>
#include <mutex>

#include "oxq_formats_more.hpp"
#include "oxq_gemv_launch.hpp"

namespace oxq {

constexpr uint32_t LMH_THREADS = 256, LMH_MAX_K = 8, LMH_MAX_BLOCKS = 512;
constexpr uint32_t LMH_TICKETS = 1024;
static __device__ uint32_t lmh_tickets[LMH_TICKETS];
static std::atomic<uint32_t> g_lmh_next_ticket{0};

template <class F, int STEPS, int RB>
__global__ __launch_bounds__(LMH_THREADS) void gemv_q8_topk(const uint8_t *__restrict__ W, const uint8_t *__restrict__ A,
                                                           float *__restrict__ out, uint32_t n_rows, uint32_t units,
                                                           size_t row_bytes, uint32_t n_cols, uint32_t k,
                                                           uint64_t *lists, uint32_t *ticket,
                                                           float *__restrict__ out_vals, uint32_t *__restrict__ out_idx) {
    __shared__ uint64_t wave_list[4][LMH_MAX_K];
    __shared__ __attribute__((aligned(16))) uint64_t all_lists[LMH_MAX_BLOCKS * LMH_MAX_K];
    const uint32_t lane = threadIdx.x & 63;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const uint32_t group = blockIdx.x * 4 + wave, n_groups = gridDim.x * 4;
    const typename F::Lane kc = F::lane_consts(lane);
    const uint32_t n_batches = (n_rows + RB - 1) / RB;

    // ---- the GEMV: one wave per row, RB rows per batch, the next batch's weights in flight while one is reduced ----
    uint64_t key[RB];
#pragma unroll
    for (int r = 0; r < RB; r++) key[r] = 0;
    if (group < n_batches) {
        typename F::Act act[STEPS];
        const ActQ8 src = ActQ8::make(A, n_cols);
#pragma unroll
        for (int s = 0; s < STEPS; s++) {
            const uint32_t u = (uint32_t)(s * 64) + lane;
            F::load_act(act[s], src, min(u, units - 1), u < units, kc);
        }
        Batch<F, STEPS, RB> b0, b1;
        load_batch<F, STEPS, RB>(b0, W, nullptr, group, n_rows, row_bytes, units, 0, lane, kc, false);
        uint32_t trip = 0;
        // lane r (< RB) holds row r's sum: store it, and keep it as a key in the lane of this trip
        auto finish = [&](float res, uint32_t batch) {
            const uint32_t row = batch * RB + lane;
            if (lane < RB && row < n_rows) out[row] = res;
#pragma unroll
            for (int r = 0; r < RB; r++) {
                const float v = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, res), r));
                const uint32_t rr = batch * RB + r;
                if (lane == trip && rr < n_rows) key[r] = topk_key(v, rr);
            }
            trip++;
        };
        uint32_t batch = group;
        while (true) {
            const uint32_t next = batch + n_groups;
            if (next >= n_batches) {
                finish(reduce_batch<F, STEPS, RB, false>(b0, act, nullptr, batch, n_rows, units, 0, 0, lane, kc), batch);
                break;
            }
            load_batch<F, STEPS, RB>(b1, W, nullptr, next, n_rows, row_bytes, units, 0, lane, kc, false);
            finish(reduce_batch<F, STEPS, RB, false>(b0, act, nullptr, batch, n_rows, units, 0, 0, lane, kc), batch);
            const uint32_t next2 = next + n_groups;
            if (next2 >= n_batches) {
                finish(reduce_batch<F, STEPS, RB, false>(b1, act, nullptr, next, n_rows, units, 0, 0, lane, kc), next);
                break;
            }
            load_batch<F, STEPS, RB>(b0, W, nullptr, next2, n_rows, row_bytes, units, 0, lane, kc, false);
            finish(reduce_batch<F, STEPS, RB, false>(b1, act, nullptr, next, n_rows, units, 0, 0, lane, kc), next);
            batch = next2;
        }
    }

    // ---- the wave's k largest, in order; then the work group's, by its first wave ----
    for (uint32_t r = 0; r < k; r++) {
        uint64_t m = key[0];
#pragma unroll
        for (int j = 1; j < RB; j++) m = max_u64(m, key[j]);
        const uint64_t best = wave_max_u64(m);
#pragma unroll
        for (int j = 0; j < RB; j++)
            if (key[j] == best) key[j] = 0;  // keys are unique (they carry the index); 0 == 0 is harmless
        if (lane == 0) wave_list[wave][r] = best;
    }
    __syncthreads();
    if (wave != 0) return;
    uint64_t mine = lane < 4 * k ? wave_list[lane / k][lane % k] : 0;
    uint64_t chosen = 0;  // lane r: the work group's r-th largest
    for (uint32_t r = 0; r < k; r++) {
        const uint64_t best = wave_max_u64(mine);
        if (mine == best) mine = 0;
        if (lane == r) chosen = best;
    }
    // one store instruction for the list, and one that goes through to memory, where the work groups of the other
    // compute dies can read it
    if (lane < k) __hip_atomic_store(&lists[(size_t)blockIdx.x * k + lane], chosen, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);

    // ---- the last work group to get here merges the lists ----
    uint32_t last = 0;
    // The list's stores have completed before the ticket is drawn, and the last work group reads the lists past its
    // own L2, after its ticket came back: no cache-wide write-back or invalidation (a device-scope fence in each of 255
    // work groups that end together cost 10 us here: every one of them walks its compute die's L2).
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    if (lane == 0) {
        last = __hip_atomic_fetch_add(ticket, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == gridDim.x - 1 ? 1u : 0u;
        // every work group has drawn: the word goes back to zero for the next launch
        if (last) __hip_atomic_store(ticket, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    if (!__builtin_amdgcn_readfirstlane((int)last)) return;
    const uint32_t n_lists = gridDim.x, n_cand = n_lists * k;
    for (uint32_t j0 = 0; j0 < n_cand; j0 += 512) {  // eight independent loads per lane and trip
        uint64_t v[8];
#pragma unroll
        for (uint32_t u = 0; u < 8; u++)
            v[u] = j0 + u * 64 + lane < n_cand ? __hip_atomic_load(&lists[j0 + u * 64 + lane], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) : 0;
#pragma unroll
        for (uint32_t u = 0; u < 8; u++)
            if (j0 + u * 64 + lane < n_cand) all_lists[j0 + u * 64 + lane] = v[u];
    }
    // lane l walks lists l, l + 64, ...: their heads in registers, the next key of a list from LDS when its head wins
    constexpr uint32_t PER_LANE = LMH_MAX_BLOCKS / 64;
    uint32_t head[PER_LANE];
    uint64_t cur[PER_LANE];
#pragma unroll
    for (uint32_t j = 0; j < PER_LANE; j++) {
        head[j] = 0;
        cur[j] = lane + 64 * j < n_lists ? all_lists[(size_t)(lane + 64 * j) * k] : 0;
    }
    for (uint32_t r = 0; r < k; r++) {
        uint64_t m = cur[0];
#pragma unroll
        for (uint32_t j = 1; j < PER_LANE; j++) m = max_u64(m, cur[j]);
        const uint64_t best = wave_max_u64(m);
#pragma unroll
        for (uint32_t j = 0; j < PER_LANE; j++)
            if (cur[j] == best && best != 0) {
                head[j]++;
                cur[j] = head[j] < k ? all_lists[(size_t)(lane + 64 * j) * k + head[j]] : 0;
            }
        if (lane == r) chosen = best;
    }
    if (lane < k) {
        out_vals[lane] = topk_value(chosen);
        out_idx[lane] = 0xFFFFFFFFu - (uint32_t)chosen;
    }
}

// The ticket words of the current device (each device holds its own copy of the array).
static uint32_t *lmh_ticket_base() {
    static std::mutex mu;
    static uint32_t *base[64] = {};
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return nullptr;
    std::lock_guard<std::mutex> lock(mu);
    if (!base[dev] && hipGetSymbolAddress(reinterpret_cast<void **>(&base[dev]), HIP_SYMBOL(lmh_tickets)) != hipSuccess)
        base[dev] = nullptr;
    return base[dev];
}

struct LmhPlan {
    uint32_t steps = 0, rb = 0, blocks = 0;
    size_t row_bytes = 0;
    uint32_t units = 0;
};

// The launch gemv_q8_cached would get for this matrix (oxq_gemv_launch.hpp), if it is one the kernel above covers: one
// wave per row of at most two 64-lane steps, at most 64 row batches per wave, at most 512 work groups (their lists
// in the last one's LDS), k <= 8.
template <class F>
static bool lmh_plan(uint32_t n_rows, uint32_t n_cols, uint32_t k, LmhPlan &p) {
    if (n_cols == 0 || n_cols % F::BLOCK_COLS != 0 || n_rows < k || k == 0 || k > LMH_MAX_K) return false;
    p.units = n_cols / F::UNIT_COLS;
    p.row_bytes = (size_t)(n_cols / F::BLOCK_COLS) * F::BLOCK_BYTES;
    p.steps = (p.units + 63) / 64;
    if (p.steps > 2) return false;
    p.rb = p.row_bytes <= F::TWO_ROW_BATCH_BYTES ? 2 : 1;
    GemvArgs a;
    a.waves_per_cu = 0;
    const uint32_t width = launch_width<F>(a, (uint64_t)n_rows * p.row_bytes);
    const uint32_t n_batches = (n_rows + p.rb - 1) / p.rb;
    uint32_t max_groups = device_cus() * width;
    if (max_groups == 0) max_groups = 1;
    const uint32_t passes = (n_batches + max_groups - 1) / max_groups;
    const uint32_t groups = (n_batches + passes - 1) / passes;
    p.blocks = (groups + 3) / 4;
    if (p.blocks == 0) p.blocks = 1;
    const uint32_t trips = (n_batches + p.blocks * 4 - 1) / (p.blocks * 4);
    return trips <= 64 && p.blocks <= LMH_MAX_BLOCKS;
}

template <class F, int STEPS, int RB>
static hipError_t lmh_launch(const LmhPlan &p, const uint8_t *W, const uint8_t *A, float *out, uint32_t n_rows,
                             uint32_t n_cols, uint32_t k, uint64_t *lists, float *out_vals, uint32_t *out_idx,
                             hipStream_t stream) {
    uint32_t *const base = lmh_ticket_base();
    if (!base) return hipErrorInvalidDevice;
    uint32_t *const ticket = base + g_lmh_next_ticket.fetch_add(1, std::memory_order_relaxed) % LMH_TICKETS;
    auto kern = &gemv_q8_topk<F, STEPS, RB>;
    note_launch("gemv_q8_topk", F::TYPE_ID, STEPS, RB, 1, 0, p.blocks, 1, LMH_THREADS);
    hipLaunchKernelGGL(kern, dim3(p.blocks), dim3(LMH_THREADS), 0, stream, W, A, out, n_rows, p.units, p.row_bytes, n_cols, k,
                       lists, ticket, out_vals, out_idx);
    return hipGetLastError();
}

template <class F>
static hipError_t lmh_format(const uint8_t *W, const uint8_t *A, float *out, uint32_t n_rows, uint32_t n_cols, uint32_t k,
                             uint64_t *lists, float *out_vals, uint32_t *out_idx, hipStream_t stream) {
    LmhPlan p;
    if (!lmh_plan<F>(n_rows, n_cols, k, p)) return hipErrorNotSupported;
#define OXQ_LMH(ST, RBV) return lmh_launch<F, ST, RBV>(p, W, A, out, n_rows, n_cols, k, lists, out_vals, out_idx, stream)
    if (p.steps == 1) {
        if (p.rb == 2) OXQ_LMH(1, 2);
        OXQ_LMH(1, 1);
    }
    if (p.rb == 2) OXQ_LMH(2, 2);
    OXQ_LMH(2, 1);
#undef OXQ_LMH
}

// Bytes of the lists for this shape, 0 where the one-launch form does not apply (the caller then runs the GEMV and
// the top-k launches).
size_t lm_head_topk_lists_bytes(uint32_t type, uint32_t n_rows, uint32_t n_cols, uint32_t k) {
    LmhPlan p;
    bool ok = false;
    switch (type) {
    case OXQ_TYPE_Q6_K: ok = lmh_plan<FmtQ6K>(n_rows, n_cols, k, p); break;
    case OXQ_TYPE_Q8_0: ok = lmh_plan<FmtQ8_0>(n_rows, n_cols, k, p); break;
    case OXQ_TYPE_Q4_K: ok = lmh_plan<FmtQ4K>(n_rows, n_cols, k, p); break;
    case OXQ_TYPE_Q5_K: ok = lmh_plan<FmtQ5K>(n_rows, n_cols, k, p); break;
    case OXQ_TYPE_Q4_0: ok = lmh_plan<FmtQ4_0>(n_rows, n_cols, k, p); break;
    default: break;
    }
    return ok ? (size_t)p.blocks * k * sizeof(uint64_t) : 0;
}

hipError_t launch_lm_head_topk(uint32_t type, const uint8_t *W, const uint8_t *A, float *out, uint32_t n_rows, uint32_t n_cols,
                               uint32_t k, void *lists, float *out_vals, uint32_t *out_idx, hipStream_t stream) {
    uint64_t *const l = static_cast<uint64_t *>(lists);
    switch (type) {
    case OXQ_TYPE_Q6_K: return lmh_format<FmtQ6K>(W, A, out, n_rows, n_cols, k, l, out_vals, out_idx, stream);
    case OXQ_TYPE_Q8_0: return lmh_format<FmtQ8_0>(W, A, out, n_rows, n_cols, k, l, out_vals, out_idx, stream);
    case OXQ_TYPE_Q4_K: return lmh_format<FmtQ4K>(W, A, out, n_rows, n_cols, k, l, out_vals, out_idx, stream);
    case OXQ_TYPE_Q5_K: return lmh_format<FmtQ5K>(W, A, out, n_rows, n_cols, k, l, out_vals, out_idx, stream);
    case OXQ_TYPE_Q4_0: return lmh_format<FmtQ4_0>(W, A, out, n_rows, n_cols, k, l, out_vals, out_idx, stream);
    default: return hipErrorNotSupported;
    }
}

}  // namespace oxq
