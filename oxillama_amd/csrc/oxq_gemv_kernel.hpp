// Kernel templates of the Q8_0-activation GEMV (see oxq_gemv.hip for the design).
#pragma once
#include <type_traits>

#include "oxq_formats.hpp"
#include "oxq_q8_encode.hpp"

namespace oxq {

// Cached-activation kernel.  A work group is four waves.  KS waves share a row
// (wave `part` owns steps [part*STEPS, (part+1)*STEPS) of it, i.e. a contiguous
// slice of the columns) and 4/KS such groups work on different rows.  The
// activation constants of a wave's steps live in registers for the whole kernel.
// Rows are taken in batches of RB; the weight loads of the next batch are issued
// (into a second register set) before the current batch is reduced, so every
// wave always has loads in flight.  With KS > 1 the per-wave row sums are added
// through LDS in a fixed order (part 0, 1, ...), one barrier per batch.
// SRC says where the activations come from: Q8_0 blocks in memory (ActQ8), or an fp32
// vector that the work group quantizes into LDS first (ActF32).  blockIdx.y selects one
// of up to four matrices of the same shape that share the activations.
template <class F, int STEPS, int RB>
struct Batch {
    typename F::Wt w[RB][STEPS];
    float old;
};

template <class F, int STEPS, int RB>
__device__ __forceinline__ void load_batch(Batch<F, STEPS, RB> &b, const uint8_t *__restrict__ W,
                                           const float *__restrict__ old, uint32_t batch, uint32_t n_rows,
                                           size_t row_bytes, uint32_t units, uint32_t unit0, uint32_t lane,
                                           const typename F::Lane &k, bool want_old) {
    const uint32_t row0 = batch * RB;
    b.old = 0.0f;
    if (want_old && lane < RB && row0 + lane < n_rows) b.old = old[row0 + lane];
#pragma unroll
    for (int r = 0; r < RB; r++) {
        const uint32_t row = min(row0 + r, n_rows - 1);  // past the last row: re-read it, result unused
        const uint8_t *rp = W + (size_t)row * row_bytes;
#pragma unroll
        for (int s = 0; s < STEPS; s++) {
            const uint32_t u = min(unit0 + (uint32_t)(s * 64) + lane, units - 1);  // past the end: last unit
            F::load_w(b.w[r][s], rp, u, k);
        }
    }
}

// Lane r (r < RB) returns the wave's sum for row r of the batch.
template <class F, int STEPS, int RB, bool DUMP>
__device__ __forceinline__ float reduce_batch(const Batch<F, STEPS, RB> &b, const typename F::Act (&act)[STEPS],
                                              int32_t *__restrict__ sums, uint32_t batch, uint32_t n_rows,
                                              uint32_t units, uint32_t unit0, uint32_t groups_per_row, uint32_t lane,
                                              const typename F::Lane &k) {
    const uint32_t row0 = batch * RB;
    float res = 0.0f;
#pragma unroll
    for (int r = 0; r < RB; r++) {
        const uint32_t row = min(row0 + r, n_rows - 1);
        float acc = 0.0f;
#pragma unroll
        for (int s = 0; s < STEPS; s++) {
            const uint32_t u = unit0 + (uint32_t)(s * 64) + lane;
            acc += F::template dot<DUMP>(b.w[r][s], act[s], k, DUMP ? sums + (size_t)row * groups_per_row : nullptr, u,
                                         u < units);
        }
        const float total = wave_sum(acc);
        if (lane == (uint32_t)r) res = total;
    }
    return res;
}

// PH (measurement only): every wave writes three timestamps of the 100 MHz wall clock to `phases` --
// kernel entry, its first row batch stored, its last -- and where it ran (phase_where) at
// [(blockIdx.y * gridDim.x + blockIdx.x) * 4 + wave][4].
// Where a wave runs: XCC_ID register in the high word, HW_ID (wave, SIMD, CU, shader array, shader engine) in the low.
__device__ __forceinline__ uint64_t phase_where() {
    const uint32_t hw = __builtin_amdgcn_s_getreg((31 << 11) | 4), xcc = __builtin_amdgcn_s_getreg((31 << 11) | 20);
    return ((uint64_t)xcc << 32) | hw;
}
template <class F, class SRC, int STEPS, int RB, int KS, bool DUMP, bool PH = false>
__global__ __launch_bounds__(256) void gemv_q8_cached(const uint8_t *__restrict__ W0, const uint8_t *__restrict__ W1,
                                                     const uint8_t *__restrict__ W2, const uint8_t *__restrict__ W3,
                                                     float *__restrict__ out0, float *__restrict__ out1,
                                                     float *__restrict__ out2, float *__restrict__ out3,
                                                     const float *__restrict__ old0, const float *__restrict__ old1,
                                                     const float *__restrict__ old2, const float *__restrict__ old3,
                                                     const void *__restrict__ A, int32_t *__restrict__ sums,
                                                     uint32_t n_rows0, uint32_t n_rows1, uint32_t n_rows2,
                                                     uint32_t n_rows3, uint32_t units, uint32_t groups_per_row,
                                                     size_t row_bytes, uint32_t n_cols, uint64_t *__restrict__ phases,
                                                     const int32_t *__restrict__ group_offsets, uint32_t n_groups_e,
                                                     size_t w_stride, size_t a_stride) {
    static_assert(KS == 1 || KS == 2 || KS == 4, "waves per row");
    uint64_t ph_t0 = 0, ph_t1 = 0;
    if constexpr (PH) ph_t0 = wall_clock64();
    // Up to four matrices of one format and row length that share the activation vector (wq/wk/wv,
    // ffn_gate/ffn_up) ride in one launch: blockIdx.y picks the matrix, and each matrix gets
    // its own gridDim.x work groups (sized for the one with the most rows).  old = the vector a
    // row's sum is added to (the output itself when accumulating, a bias vector), or null.
    const uint32_t mat = blockIdx.y;
    const uint8_t *__restrict__ W = mat == 0 ? W0 : mat == 1 ? W1 : mat == 2 ? W2 : W3;
    float *__restrict__ out = mat == 0 ? out0 : mat == 1 ? out1 : mat == 2 ? out2 : out3;
    const float *__restrict__ old = mat == 0 ? old0 : mat == 1 ? old1 : mat == 2 ? old2 : old3;
    uint32_t n_rows = mat == 0 ? n_rows0 : mat == 1 ? n_rows1 : mat == 2 ? n_rows2 : n_rows3;
    if (group_offsets) {
        // Grouped form: blockIdx.y is a token row p; its group e (an expert) is the number of groups that end at or
        // before p (one load per lane and a ballot per 64 groups).  Matrix e, activation row p, output row p.
        const uint32_t ln = threadIdx.x & 63;
        uint32_t below = 0;
        for (uint32_t base = 0; base < n_groups_e; base += 64) {  // (64 groups per ballot)
            const int32_t end = base + ln < n_groups_e ? group_offsets[base + ln + 1] : 0x7FFFFFFF;
            below += (uint32_t)__builtin_popcountll(__ballot(end <= (int32_t)mat));
        }
        const uint32_t e = min(below, n_groups_e - 1);
        W = W0 + (size_t)e * w_stride;
        A = static_cast<const uint8_t *>(A) + (size_t)mat * a_stride;
        out = out0 + (size_t)mat * n_rows0;
        old = old0 ? old0 + (size_t)mat * n_rows0 : nullptr;
        n_rows = n_rows0;
    }
    constexpr uint32_t G = 4 / KS;  // row groups per work group
    __shared__ float part_sums[2][4][4];
    const uint32_t lane = threadIdx.x & 63;
    const uint32_t wave_in_wg = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const uint32_t part = wave_in_wg % KS, grp = wave_in_wg / KS;
    const uint32_t group = blockIdx.x * G + grp;
    const uint32_t n_groups = gridDim.x * G;
    const uint32_t unit0 = part * STEPS * 64;
    const typename F::Lane k = F::lane_consts(lane);
    const uint32_t n_batches = (n_rows + RB - 1) / RB;
    // With KS > 1 every wave of the work group runs the same number of trips (barriers);
    // trips past the last batch re-read the last rows and store nothing.
    const uint32_t n_trips = KS == 1 ? n_batches : ((n_batches + n_groups - 1) / n_groups) * n_groups;
    const bool want_old = old != nullptr && part == 0;
    constexpr bool F32 = std::is_same<SRC, ActF32>::value;
    Batch<F, STEPS, RB> b0, b1;
    typename F::Act act[STEPS];
    extern __shared__ uint32_t lds_acts[];  // fp32 source: [n_blocks * 8] payload dwords, then n_blocks f16 scales
    auto load_acts = [&](const auto &src) {
#pragma unroll
        for (int s = 0; s < STEPS; s++) {
            const uint32_t u = unit0 + (uint32_t)(s * 64) + lane;
            F::load_act(act[s], src, min(u, units - 1), u < units, k);  // all-zero constants past the end
        }
    };
    if constexpr (F32) {
        // fp32 activations: request the first weights, then the work group quantizes the vector into
        // LDS once (every wave takes part in the barrier) and each wave picks up its slice.
        load_batch<F, STEPS, RB>(b0, W, old, min(group, n_batches - 1), n_rows, row_bytes, units, unit0, lane, k,
                                 want_old);
        const uint32_t nb = units * (F::UNIT_COLS / 32);
        uint16_t *lds_d = reinterpret_cast<uint16_t *>(lds_acts + (size_t)nb * 8);
        quantize_to_lds(static_cast<const float *>(A), nb, n_cols, lds_acts, lds_d);
        __syncthreads();
        if (KS == 1 && group >= n_batches) return;
        load_acts(ActLds{reinterpret_cast<const u32x4 *>(lds_acts), lds_d});
    } else {
        if (KS == 1 && group >= n_batches) return;
        // Activations first (they sit in L2 and arrive early), then the first batch of
        // weights: the activation constants are derived while HBM is being read.
        load_acts(SRC::make(A, n_cols));
        load_batch<F, STEPS, RB>(b0, W, old, min(group, n_batches - 1), n_rows, row_bytes, units, unit0, lane, k,
                                 want_old);
    }

    uint32_t trip = 0;
    auto ph_done = [&]() {
        if constexpr (PH) {
            if (lane == 0) {
                uint64_t *p = phases + ((size_t)(blockIdx.y * gridDim.x + blockIdx.x) * 4 + wave_in_wg) * 4;
                p[0] = ph_t0;
                p[1] = ph_t1;
                p[2] = wall_clock64();
                p[3] = phase_where();
            }
        }
    };
    auto finish = [&](float res, float old, uint32_t batch) {
        const uint32_t row = batch * RB + lane;
        if (KS == 1) {
            if (lane < RB && row < n_rows) out[row] = old + res;
        } else {
            if (lane < RB) part_sums[trip & 1][wave_in_wg][lane] = res;
            __syncthreads();
            if (part == 0 && lane < RB && batch < n_batches && row < n_rows) {
                float t = part_sums[trip & 1][grp * KS][lane];
#pragma unroll
                for (int p = 1; p < KS; p++) t += part_sums[trip & 1][grp * KS + p][lane];
                out[row] = old + t;
            }
            trip++;
        }
        if constexpr (PH) {
            if (ph_t1 == 0) ph_t1 = wall_clock64();
        }
    };

    // Each reduce_batch call site has a fixed set of loads in flight behind it, so the
    // compiler can wait for exactly the batch it needs and leave the prefetch outstanding.
    uint32_t batch = group;
    while (true) {
        const uint32_t next = batch + n_groups;
        if (next >= n_trips) {
            const float r0 = reduce_batch<F, STEPS, RB, DUMP>(b0, act, sums, min(batch, n_batches - 1), n_rows, units,
                                                              unit0, groups_per_row, lane, k);
            finish(r0, b0.old, batch);
            ph_done();
            break;
        }
        load_batch<F, STEPS, RB>(b1, W, old, min(next, n_batches - 1), n_rows, row_bytes, units, unit0, lane, k, want_old);
        const float r0 = reduce_batch<F, STEPS, RB, DUMP>(b0, act, sums, min(batch, n_batches - 1), n_rows, units, unit0,
                                                          groups_per_row, lane, k);
        finish(r0, b0.old, batch);
        const uint32_t next2 = next + n_groups;
        if (next2 >= n_trips) {
            const float r1 = reduce_batch<F, STEPS, RB, DUMP>(b1, act, sums, min(next, n_batches - 1), n_rows, units,
                                                              unit0, groups_per_row, lane, k);
            finish(r1, b1.old, next);
            ph_done();
            break;
        }
        load_batch<F, STEPS, RB>(b0, W, old, min(next2, n_batches - 1), n_rows, row_bytes, units, unit0, lane, k, want_old);
        const float r1 = reduce_batch<F, STEPS, RB, DUMP>(b1, act, sums, min(next, n_batches - 1), n_rows, units, unit0,
                                                          groups_per_row, lane, k);
        finish(r1, b1.old, next);
        batch = next2;
    }
}

// ffn_gate and ffn_up of the dense feed-forward block (crates/oxillama-arch/src/llama/model.rs:295-310)
// with SwiGLU (swiglu.rs:15-21) and the Q8_0 quantizer of the down projection's input
// (quantize.rs:58) in the same kernel.  A work group owns rows 32b..32b+31 of BOTH matrices -- one
// Q8_0 block of h -- so nothing crosses work groups: wave w streams rows 8w..8w+7 of gate, then of
// up (RB rows per batch, the next batch's loads in flight while one is reduced; one wave per row,
// so the sums are those of gemv_q8_cached with KS = 1, bit for bit), the 64 sums meet in LDS and
// eight lanes encode the block.  h_out (optional) receives h in fp32.
// GRP: the grouped (mixture-of-experts) form for a handful of token rows -- blockIdx.y is a token row p, its expert e
// the group of group_offsets that holds p (found as in gemv_q8_cached); gate matrix Wg + e * wg_stride, up matrix
// Wu + e * wu_stride, activation row A + p * a_stride, block of h at hq + p * hq_stride.  The arguments after
// `phases` are read in that form only.
template <class F, int STEPS, int RB, int WAVES, bool PH = false, bool GRP = false>
__global__ __launch_bounds__(64 * WAVES) void gemv_q8_gate_up_swiglu(const uint8_t *__restrict__ Wg,
                                                             const uint8_t *__restrict__ Wu,
                                                             const void *__restrict__ A, uint8_t *__restrict__ hq,
                                                             float *__restrict__ h_out, uint32_t n_rows, uint32_t units,
                                                             size_t row_bytes, uint64_t *__restrict__ phases,
                                                             const int32_t *__restrict__ group_offsets,
                                                             uint32_t n_groups_e, size_t wg_stride, size_t wu_stride,
                                                             size_t a_stride, size_t hq_stride) {
    static_assert((RB == 1 || RB == 2) && (WAVES == 4 || WAVES == 8), "configuration");
    uint64_t ph_t0 = 0, ph_t1 = 0;
    if constexpr (PH) ph_t0 = wall_clock64();
    if constexpr (GRP) {
        const uint32_t p = blockIdx.y, ln = threadIdx.x & 63;
        uint32_t below = 0;
        for (uint32_t base = 0; base < n_groups_e; base += 64) {  // (64 groups per ballot)
            const int32_t end = base + ln < n_groups_e ? group_offsets[base + ln + 1] : 0x7FFFFFFF;
            below += (uint32_t)__builtin_popcountll(__ballot(end <= (int32_t)p));
        }
        const uint32_t e = min(below, n_groups_e - 1);
        Wg += (size_t)e * wg_stride;
        Wu += (size_t)e * wu_stride;
        A = static_cast<const uint8_t *>(A) + (size_t)p * a_stride;
        hq += (size_t)p * hq_stride;
        if (h_out) h_out += (size_t)p * n_rows;
    }
    constexpr int RPW = 32 / WAVES;  // rows of each matrix per wave
    constexpr int NB = RPW / RB;     // batches per matrix and wave
    __shared__ float row_sums[2][32];
    const uint32_t lane = threadIdx.x & 63;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const typename F::Lane k = F::lane_consts(lane);
    typename F::Act act[STEPS];
    {
        const auto src = ActQ8{static_cast<const uint8_t *>(A)};
#pragma unroll
        for (int s = 0; s < STEPS; s++) {
            const uint32_t u = (uint32_t)(s * 64) + lane;
            F::load_act(act[s], src, min(u, units - 1), u < units, k);
        }
    }
    const uint32_t batch0 = (blockIdx.x * 32 + wave * RPW) / RB;
    constexpr int AHEAD = 2;  // batches requested ahead of the one being reduced
    Batch<F, STEPS, RB> b[AHEAD + 1];
#pragma unroll
    for (int i = 0; i < AHEAD; i++)
        load_batch<F, STEPS, RB>(b[i], i < NB ? Wg : Wu, nullptr, batch0 + i % NB, n_rows, row_bytes, units, 0, lane, k, false);
#pragma unroll
    for (int i = 0; i < 2 * NB; i++) {
        if (i + AHEAD < 2 * NB)
            load_batch<F, STEPS, RB>(b[(i + AHEAD) % (AHEAD + 1)], i + AHEAD < NB ? Wg : Wu, nullptr,
                                     batch0 + (i + AHEAD) % NB, n_rows, row_bytes, units, 0, lane, k, false);
        const float r = reduce_batch<F, STEPS, RB, false>(b[i % (AHEAD + 1)], act, nullptr, batch0 + i % NB, n_rows, units,
                                                          0, 0, lane, k);
        if (lane < RB) row_sums[i / NB][wave * RPW + (i % NB) * RB + lane] = r;
        if constexpr (PH) {
            if (i == 0) ph_t1 = wall_clock64();
        }
    }
    if constexpr (PH) {
        if (lane == 0) {  // the wave's rows are summed: what follows is the block's SwiGLU and encode
            uint64_t *p = phases + ((size_t)blockIdx.x * WAVES + wave) * 4;
            p[0] = ph_t0;
            p[1] = ph_t1;
            p[2] = wall_clock64();
            p[3] = phase_where();
        }
    }
    __syncthreads();
    if (wave != 0) return;
    // one element of h per lane (the exp is a chain of double-precision operations: 32 lanes side by side, not four
    // in a row on eight lanes), then the encoder's layout: lane j of eight holds elements 4j..4j+3
    float hv;
    {
        const float g = row_sums[0][lane & 31], u = row_sums[1][lane & 31];
        const float sigmoid = 1.0f / (1.0f + expf_libm(-g));  // swiglu.rs:18
        hv = g * sigmoid * u;                                 // swiglu.rs:19
    }
    const uint32_t j = lane & 7;
    float v[4];
    for (int i = 0; i < 4; i++) v[i] = __shfl(hv, (int)(4 * j + i), 64);
    const bool writer = lane < 8;
    if (writer && h_out)
        for (int i = 0; i < 4; i++) h_out[(size_t)blockIdx.x * 32 + 4 * j + i] = v[i];
    encode_q8_0_lanes(v, writer, hq + (size_t)blockIdx.x * 34, j);
}

// Several activation vectors against one weight stream (a small decode batch): NV vectors'
// constants live in registers, every weight row is loaded once and dotted with each of them.
// RB rows per trip (double-buffered like the kernel above: the next trip's rows are requested
// before this trip's are reduced), KS waves per row.  Vector v reads its Q8_0 blocks at
// A + v * a_stride and writes out[v * out_stride + row].
template <class F, int STEPS, int KS, int NV, int RB>
__global__ __launch_bounds__(256) void gemv_q8_vecs(const uint8_t *__restrict__ W, const uint8_t *__restrict__ A,
                                                   size_t a_stride, float *__restrict__ out, size_t out_stride,
                                                   uint32_t n_rows, uint32_t units, size_t row_bytes,
                                                   int accumulate, uint32_t n_vecs, const float *__restrict__ bias) {
    static_assert((KS == 1 || KS == 4) && NV >= 2 && NV <= 4 && (RB == 1 || RB == 2), "configuration");
    // n_vecs <= NV: the surplus slots repeat the last vector (same loads, same stored values)
    constexpr uint32_t G = 4 / KS;
    __shared__ float part_sums[2][4][RB * 4];
    const uint32_t lane = threadIdx.x & 63;
    const uint32_t wave_in_wg = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const uint32_t part = wave_in_wg % KS, grp = wave_in_wg / KS;
    const uint32_t group = blockIdx.x * G + grp;
    const uint32_t n_groups = gridDim.x * G;
    const uint32_t unit0 = part * STEPS * 64;
    const typename F::Lane k = F::lane_consts(lane);
    const uint32_t n_batches = (n_rows + RB - 1) / RB;
    const uint32_t n_trips = KS == 1 ? n_batches : ((n_batches + n_groups - 1) / n_groups) * n_groups;
    if (KS == 1 && group >= n_batches) return;

    typename F::Act act[NV][STEPS];
#pragma unroll
    for (int v = 0; v < NV; v++)
#pragma unroll
        for (int s = 0; s < STEPS; s++) {
            const uint32_t u = unit0 + (uint32_t)(s * 64) + lane;
            F::load_act(act[v][s], ActQ8{A + (size_t)min((uint32_t)v, n_vecs - 1) * a_stride}, min(u, units - 1),
                        u < units, k);
        }
    auto load_rows = [&](typename F::Wt (&w)[RB][STEPS], uint32_t batch) {
#pragma unroll
        for (int r = 0; r < RB; r++) {
            // past the end: re-read the last row
            const uint8_t *rp = W + (size_t)min(batch * RB + (uint32_t)r, n_rows - 1) * row_bytes;
#pragma unroll
            for (int s = 0; s < STEPS; s++)
                F::load_w(w[r][s], rp, min(unit0 + (uint32_t)(s * 64) + lane, units - 1), k);
        }
    };
    uint32_t trip = 0;
    // lane r * NV + v ends up with the sum of row r of the batch against vector v
    auto reduce_rows = [&](const typename F::Wt (&w)[RB][STEPS], uint32_t batch) {
        float res = 0.0f;
#pragma unroll
        for (int r = 0; r < RB; r++)
#pragma unroll
            for (int v = 0; v < NV; v++) {
                float acc = 0.0f;
#pragma unroll
                for (int s = 0; s < STEPS; s++) {
                    const uint32_t u = unit0 + (uint32_t)(s * 64) + lane;
                    acc += F::template dot<false>(w[r][s], act[v][s], k, nullptr, u, u < units);
                }
                const float total = wave_sum(acc);
                if (lane == (uint32_t)(r * NV + v)) res = total;
            }
        const uint32_t row = batch * RB + lane / NV, vec = min(lane % NV, n_vecs - 1);
        if (KS == 1) {
            if (lane < RB * NV && row < n_rows) {
                float *o = out + (size_t)vec * out_stride + row;
                *o = (accumulate ? *o : bias ? bias[row] : 0.0f) + res;
            }
        } else {
            if (lane < RB * NV) part_sums[trip & 1][wave_in_wg][lane] = res;
            __syncthreads();
            if (part == 0 && lane < RB * NV && batch < n_batches && row < n_rows) {
                float t = part_sums[trip & 1][grp * KS][lane];
#pragma unroll
                for (int p = 1; p < KS; p++) t += part_sums[trip & 1][grp * KS + p][lane];
                float *o = out + (size_t)vec * out_stride + row;
                *o = (accumulate ? *o : bias ? bias[row] : 0.0f) + t;
            }
            trip++;
        }
    };

    typename F::Wt w0[RB][STEPS], w1[RB][STEPS];
    load_rows(w0, min(group, n_batches - 1));
    uint32_t batch = group;
    while (true) {
        const uint32_t next = batch + n_groups;
        if (next >= n_trips) {
            reduce_rows(w0, batch);
            break;
        }
        load_rows(w1, min(next, n_batches - 1));
        reduce_rows(w0, batch);
        const uint32_t next2 = next + n_groups;
        if (next2 >= n_trips) {
            reduce_rows(w1, next);
            break;
        }
        load_rows(w0, min(next2, n_batches - 1));
        reduce_rows(w1, next);
        batch = next2;
    }
}

// Any number of steps: activations re-read (from L2) for every row.  Also the kernel of rows that end
// inside a block (n_cols not a whole number of blocks): the columns past n_cols are skipped.
template <class F, bool DUMP>
__global__ __launch_bounds__(256) void gemv_q8_generic(const uint8_t *__restrict__ W,
                                                      const uint8_t *__restrict__ A,
                                                      float *__restrict__ out, int32_t *__restrict__ sums,
                                                      uint32_t n_rows, uint32_t units, uint32_t groups_per_row,
                                                      size_t row_bytes, const float *__restrict__ old, uint32_t n_cols) {
    const uint32_t lane = threadIdx.x & 63;
    const uint32_t wave = __builtin_amdgcn_readfirstlane((blockIdx.x * blockDim.x + threadIdx.x) >> 6);
    const uint32_t n_waves = (gridDim.x * blockDim.x) >> 6;
    const typename F::Lane k = F::lane_consts(lane);
    const uint32_t steps = (units + 63) / 64;
    for (uint32_t row = wave; row < n_rows; row += n_waves) {
        const uint8_t *rp = W + (size_t)row * row_bytes;
        float acc = 0.0f;
        for (uint32_t s = 0; s < steps; s++) {
            const uint32_t u = s * 64 + lane;
            const bool valid = u < units;
            typename F::Act a;
            typename F::Wt w;
            const uint32_t uc = min(u, units - 1);
            F::load_w(w, rp, uc, k);
            F::load_act(a, ActQ8Tail{A, n_cols}, uc, valid, k);
            acc += F::template dot<DUMP>(w, a, k, DUMP ? sums + (size_t)row * groups_per_row : nullptr, u, valid);
        }
        const float total = wave_sum(acc);
        if (lane == 0) out[row] = (old ? old[row] : 0.0f) + total;
    }
}

}  // namespace oxq
