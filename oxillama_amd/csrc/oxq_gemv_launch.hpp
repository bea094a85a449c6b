// Launch policy of the GEMV kernels, as templates over the format policy: shared by the
// translation units that instantiate them for their formats.
#pragma once
#include "oxq_gemv_kernel.hpp"
#include "oxq_internal.hpp"

namespace oxq {

// Launch width when the caller names none: 8 resident waves per compute unit unless the format's
// policy says otherwise (WAVES_PER_CU).
template <class F, class = void> struct format_waves_per_cu { static constexpr uint32_t value = 8; };
template <class F> struct format_waves_per_cu<F, std::void_t<decltype(F::WAVES_PER_CU)>> {
    static constexpr uint32_t value = F::WAVES_PER_CU;
};
// Formats whose GEMV kernels also exist in the timestamping instantiation (the BASELINE decode shapes).
template <class F> struct phase_probe_format {
    static constexpr bool value = F::TYPE_ID == OXQ_TYPE_Q4_K || F::TYPE_ID == OXQ_TYPE_Q6_K || F::TYPE_ID == OXQ_TYPE_Q8_0 ||
                                  F::TYPE_ID == OXQ_TYPE_Q4_0;
};

// A launch over at most this many weight bytes is "small": it ends within a few microseconds, most of which are the
// ramp of its waves, and runs faster on fewer, longer-lived waves (measured on MI355X at 4096 x 4096 and 6144 x 4096:
// 3-7 % faster with one work group per compute unit than with two; from 14336 x 4096 on the wider launch wins).
constexpr uint64_t SMALL_LAUNCH_BYTES = 28ull << 20;

template <class F>
static uint32_t launch_width(const GemvArgs &a, uint64_t weight_bytes) {
    if (a.waves_per_cu) return a.waves_per_cu;
    const uint32_t w = format_waves_per_cu<F>::value;
    return weight_bytes <= SMALL_LAUNCH_BYTES && w > 4 ? 4 : w;
}

template <class F, class SRC, int STEPS, int RB, int KS, bool DUMP>
static hipError_t launch_cached_src(const GemvArgs &a, uint32_t units, uint32_t groups_per_row, size_t row_bytes,
                                hipStream_t stream) {
    constexpr uint32_t G = 4 / KS;  // row groups per work group
    const uint32_t n_mats = a.group_offsets ? a.n_pairs : a.n_mats ? a.n_mats : 1;
    const uint8_t *w[4];
    float *o[4];
    const float *old[4];  // what a row's sum is added to: the output (accumulate), a bias, or nothing
    uint32_t rows[4];
    uint32_t max_rows = a.n_rows;
    for (uint32_t i = 0; i < 4; i++) {
        const bool more = i > 0 && i < n_mats && !a.group_offsets;
        w[i] = more ? a.W_more[i - 1] : a.W;
        o[i] = more ? a.out_more[i - 1] : a.out;
        old[i] = a.accumulate ? o[i] : more ? a.bias_more[i - 1] : a.bias;
        rows[i] = more && a.n_rows_more[i - 1] ? a.n_rows_more[i - 1] : a.n_rows;
        if (rows[i] > max_rows) max_rows = rows[i];
    }
    const uint32_t n_batches = (max_rows + RB - 1) / RB;
    // the launch width is shared by the matrices of the call
    uint64_t total_rows = 0;
    for (uint32_t i = 0; i < n_mats; i++) total_rows += rows[i < 4 ? i : 0];
    // each matrix gets gridDim.x work groups, sized so that the whole launch fills the chip once
    // (several matrices in one launch keep the format's width: not measured otherwise)
    const uint32_t width = launch_width<F>(a, n_mats == 1 ? total_rows * row_bytes : ~0ull);
    uint32_t max_groups = (uint32_t)((uint64_t)(device_cus() * width / KS) * max_rows / (total_rows ? total_rows : 1));
    if (max_groups == 0) max_groups = 1;
    // Equal share per group: ceil(n_batches / passes) groups, each doing `passes` batches.
    const uint32_t passes = (n_batches + max_groups - 1) / max_groups;
    const uint32_t groups = (n_batches + passes - 1) / passes;
    uint32_t blocks = (groups + G - 1) / G;
    if (blocks == 0) blocks = 1;
    const void *acts = a.X ? static_cast<const void *>(a.X) : static_cast<const void *>(a.A);
    if constexpr (phase_probe_format<F>::value && std::is_same<SRC, ActQ8>::value && !DUMP && STEPS <= 2) {
        // measurement: the same kernel with three timestamps per wave (oxq_set_gemv_phase_probe)
        uint64_t *ph = g_phase_buf.load(std::memory_order_relaxed);
        if (ph && (size_t)blocks * n_mats * 4 * 4 * 8 <= g_phase_cap.load(std::memory_order_relaxed)) {
            hipLaunchKernelGGL((gemv_q8_cached<F, SRC, STEPS, RB, KS, DUMP, true>), dim3(blocks, n_mats), dim3(256), 0, stream,
                               w[0], w[1], w[2], w[3], o[0], o[1], o[2], o[3], old[0], old[1], old[2], old[3], acts, a.sums,
                               rows[0], rows[1], rows[2], rows[3], units, groups_per_row, row_bytes, a.n_cols, ph,
                               a.group_offsets, a.n_groups, a.w_stride, a.a_stride);
            note_launch("gemv_q8_cached_phases", F::TYPE_ID, STEPS, RB, KS, DUMP, blocks, n_mats, 256);
            return hipGetLastError();
        }
    }
    // fp32 source: LDS for the quantized vector (32 payload bytes + one f16 scale per block)
    const size_t lds = std::is_same<SRC, ActF32>::value ? (size_t)units * (F::UNIT_COLS / 32) * 34 : 0;
    note_launch(std::is_same<SRC, ActF32>::value ? "gemv_q8_cached_f32" : "gemv_q8_cached", F::TYPE_ID, STEPS, RB, KS, DUMP,
                blocks, n_mats, 256);
    hipLaunchKernelGGL((gemv_q8_cached<F, SRC, STEPS, RB, KS, DUMP>), dim3(blocks, n_mats), dim3(256), lds, stream, w[0],
                       w[1], w[2], w[3], o[0], o[1], o[2], o[3], old[0], old[1], old[2], old[3], acts, a.sums, rows[0],
                       rows[1], rows[2], rows[3], units, groups_per_row, row_bytes, a.n_cols, (uint64_t *)nullptr,
                       a.group_offsets, a.n_groups, a.w_stride, a.a_stride);
    return hipGetLastError();
}

// a.X set: fp32 activations, quantized to Q8_0 in registers by every wave (no dump variant).
template <class F, int STEPS, int RB, int KS, bool DUMP>
static hipError_t launch_cached(const GemvArgs &a, uint32_t units, uint32_t groups_per_row, size_t row_bytes,
                                hipStream_t stream) {
    if constexpr (!DUMP) {
        if (a.X) return launch_cached_src<F, ActF32, STEPS, RB, KS, false>(a, units, groups_per_row, row_bytes, stream);
    }
    return launch_cached_src<F, ActQ8, STEPS, RB, KS, DUMP>(a, units, groups_per_row, row_bytes, stream);
}

template <class F, int STEPS, int KS>
static hipError_t launch_steps(const GemvArgs &a, uint32_t units, uint32_t groups_per_row, size_t row_bytes,
                               uint32_t rb, hipStream_t stream) {
    if (a.sums) return launch_cached<F, STEPS, 1, KS, true>(a, units, groups_per_row, row_bytes, stream);
    if constexpr (STEPS <= 2) {
        if (rb >= 4) return launch_cached<F, STEPS, 4, KS, false>(a, units, groups_per_row, row_bytes, stream);
        if (rb >= 2) return launch_cached<F, STEPS, 2, KS, false>(a, units, groups_per_row, row_bytes, stream);
    }
    return launch_cached<F, STEPS, 1, KS, false>(a, units, groups_per_row, row_bytes, stream);
}

template <class F>
static hipError_t launch_format(const GemvArgs &a, uint32_t group_cols, hipStream_t stream) {
    // a row may end inside a block (the reference skips the columns past n_cols): whole blocks are
    // stored and streamed (a unit's weights need not be consecutive columns), and the activation
    // source hands out zero bytes for the columns that do not exist
    const uint32_t units = (a.n_cols + F::BLOCK_COLS - 1) / F::BLOCK_COLS * (F::BLOCK_COLS / F::UNIT_COLS);
    const uint32_t groups_per_row = a.n_cols / group_cols;
    const size_t row_bytes = (size_t)((a.n_cols + F::BLOCK_COLS - 1) / F::BLOCK_COLS) * F::BLOCK_BYTES;
    const uint32_t steps = (units + 63) / 64;
    // Long rows are split over the four waves of a work group (fewer registers per wave,
    // more waves per SIMD); short ones keep one wave per row and need no barrier.
    uint32_t ks = a.waves_per_row;
    if (ks == 0) ks = steps >= 3 ? 4 : 1;
    // Rows per batch: two while a wave's slice of a row is at most ~3.4 KB, else one
    // (measured on MI355X: more in flight per wave does not pay beyond that); Q6_K always one.
    uint32_t rb = a.rows_per_batch;
    if (rb == 0) {
        const size_t slice = row_bytes / (ks >= 4 ? 4 : 1);
        // a small launch (few trips per wave) keeps two rows in flight up to a slightly longer slice: Q8_0 at 4096 columns
        const bool small = (uint64_t)a.n_rows * row_bytes <= SMALL_LAUNCH_BYTES && a.n_mats <= 1 && !a.group_offsets;
        rb = slice <= F::TWO_ROW_BATCH_BYTES || (small && slice <= 4400) ? 2 : 1;
    }
    // Q8_0 activations and a row that ends inside a block: the kernel that masks the activations
    const bool ragged_q8 = a.n_cols % F::BLOCK_COLS != 0 && !a.X;
    if (ks >= 4 && steps <= 32 && !ragged_q8) {
        const uint32_t sw = (steps + 3) / 4;
        switch (sw) {
        case 1: return launch_steps<F, 1, 4>(a, units, groups_per_row, row_bytes, rb, stream);
        case 2: return launch_steps<F, 2, 4>(a, units, groups_per_row, row_bytes, rb, stream);
        case 3:
        case 4: return launch_steps<F, 4, 4>(a, units, groups_per_row, row_bytes, rb, stream);
        default: return launch_steps<F, 8, 4>(a, units, groups_per_row, row_bytes, rb, stream);
        }
    }
    switch (ragged_q8 ? 0 : steps) {
    case 1: return launch_steps<F, 1, 1>(a, units, groups_per_row, row_bytes, rb, stream);
    case 2: return launch_steps<F, 2, 1>(a, units, groups_per_row, row_bytes, rb, stream);
    case 3:
    case 4: return launch_steps<F, 4, 1>(a, units, groups_per_row, row_bytes, rb, stream);
    case 5:
    case 6:
    case 7:
    case 8: return launch_steps<F, 8, 1>(a, units, groups_per_row, row_bytes, rb, stream);
    default: break;
    }
    if (a.X || a.group_offsets) return hipErrorNotSupported;  // rows this long re-read the activations: Q8_0 blocks only
    const uint32_t max_waves = device_cus() * launch_width<F>(a, ~0ull);
    uint32_t waves = a.n_rows < max_waves ? a.n_rows : max_waves;
    uint32_t blocks = (waves + 3) / 4;
    if (blocks == 0) blocks = 1;
    if (a.sums)
        hipLaunchKernelGGL((gemv_q8_generic<F, true>), dim3(blocks), dim3(256), 0, stream, a.W, a.A, a.out, a.sums,
                           a.n_rows, units, groups_per_row, row_bytes, a.accumulate ? a.out : a.bias, a.n_cols);
    else
        hipLaunchKernelGGL((gemv_q8_generic<F, false>), dim3(blocks), dim3(256), 0, stream, a.W, a.A, a.out, a.sums,
                           a.n_rows, units, groups_per_row, row_bytes, a.accumulate ? a.out : a.bias, a.n_cols);
    return hipGetLastError();
}

// gate + up + SwiGLU + quantize in one launch: rows short enough for one wave per row (the
// configurations launch_format gives KS = 1 and at most two steps), a whole number of 32-row blocks.
template <class F>
static hipError_t launch_gate_up_swiglu_format(const uint8_t *Wg, const uint8_t *Wu, const uint8_t *acts, uint8_t *hq,
                                               float *h, uint32_t n_rows, uint32_t n_cols, hipStream_t stream,
                                               const GateUpGroups &grp = GateUpGroups()) {
    const uint32_t units = n_cols / F::UNIT_COLS;
    const size_t row_bytes = (size_t)(n_cols / F::BLOCK_COLS) * F::BLOCK_BYTES;
    const uint32_t steps = (units + 63) / 64;
    if (steps > 2 || n_rows % 32 != 0 || n_rows == 0) return hipErrorNotSupported;
    const bool two = row_bytes <= F::TWO_ROW_BATCH_BYTES && steps == 1;
    if (grp.offsets) {
        if (grp.n_groups > 4096 || grp.n_pairs == 0 || grp.n_pairs > 65535) return hipErrorNotSupported;
        const dim3 grid(n_rows / 32, grp.n_pairs);
        const size_t a_stride = (size_t)(n_cols / 32) * 34, hq_stride = (size_t)(n_rows / 32) * 34;
#define OXQ_LAUNCH_GRP(ST, RBV)                                                                                      \
    note_launch("gemv_q8_gate_up_swiglu_grouped", F::TYPE_ID, ST, RBV, 4, 0, grid.x, grid.y, 256);                   \
    hipLaunchKernelGGL((gemv_q8_gate_up_swiglu<F, ST, RBV, 4, false, true>), grid, dim3(256), 0, stream, Wg, Wu,    \
                       acts, hq, h, n_rows, units, row_bytes, (uint64_t *)nullptr, grp.offsets, grp.n_groups,         \
                       grp.wg_stride, grp.wu_stride, a_stride, hq_stride)
        if (steps == 1) {
            if (two) { OXQ_LAUNCH_GRP(1, 2); } else { OXQ_LAUNCH_GRP(1, 1); }
        } else {
            if (two) { OXQ_LAUNCH_GRP(2, 2); } else { OXQ_LAUNCH_GRP(2, 1); }
        }
#undef OXQ_LAUNCH_GRP
        return hipGetLastError();
    }
    const dim3 grid(n_rows / 32);
    uint64_t *ph = nullptr;
    if constexpr (phase_probe_format<F>::value) {
        ph = g_phase_buf.load(std::memory_order_relaxed);
        if (ph && (size_t)grid.x * 8 * 4 * 8 > g_phase_cap.load(std::memory_order_relaxed)) ph = nullptr;
    }
#define OXQ_LAUNCH(ST, RBV)                                                                                          \
    note_launch("gemv_q8_gate_up_swiglu", F::TYPE_ID, ST, RBV, 4, 0, grid.x, 1, 256);                                \
    if constexpr (phase_probe_format<F>::value) {                                                                    \
        if (ph) {                                                                                                    \
            hipLaunchKernelGGL((gemv_q8_gate_up_swiglu<F, ST, RBV, 4, true>), grid, dim3(256), 0, stream, Wg, Wu,    \
                               acts, hq, h, n_rows, units, row_bytes, ph, (const int32_t *)nullptr, 0u, (size_t)0,   \
                               (size_t)0, (size_t)0, (size_t)0);                                                     \
            return hipGetLastError();                                                                                \
        }                                                                                                            \
    }                                                                                                                \
    hipLaunchKernelGGL((gemv_q8_gate_up_swiglu<F, ST, RBV, 4>), grid, dim3(256), 0, stream, Wg, Wu, acts, hq, h,     \
                       n_rows, units, row_bytes, (uint64_t *)nullptr, (const int32_t *)nullptr, 0u, (size_t)0,       \
                       (size_t)0, (size_t)0, (size_t)0)
    if (steps == 1) {
        if (two) { OXQ_LAUNCH(1, 2); } else { OXQ_LAUNCH(1, 1); }
    } else {
        if (two) { OXQ_LAUNCH(2, 2); } else { OXQ_LAUNCH(2, 1); }
    }
#undef OXQ_LAUNCH
    return hipGetLastError();
}

// True when one launch can take the n_mats matrices of `a` (the register-cached kernel, whole
// batches per matrix); otherwise the caller gets one launch per matrix.
template <class F>
static bool multi_in_one_launch(const GemvArgs &a) {
    return (a.n_cols / F::UNIT_COLS + 63) / 64 <= 32 && !a.sums && (a.n_cols % F::BLOCK_COLS == 0 || a.X);
}

// ---- several activation vectors per launch -------------------------------------------------

template <class F, int STEPS, int KS, int NV>
static hipError_t launch_vecs_k(const GemvVecsArgs &a, uint32_t units, size_t row_bytes, hipStream_t stream) {
    constexpr uint32_t G = 4 / KS;
    // Two rows per trip where a wave's slice of a row is one step (measured on 14336 x 4096 and 4096 x 14336:
    // one row per trip leaves too few bytes in flight per wave)
    constexpr int RB = STEPS == 1 ? 2 : 1;
    const uint32_t n_batches = (a.n_rows + RB - 1) / RB;
    const uint32_t max_groups = device_cus() * 8 / KS;
    const uint32_t passes = (n_batches + max_groups - 1) / max_groups;
    const uint32_t groups = (n_batches + passes - 1) / passes;
    uint32_t blocks = (groups + G - 1) / G;
    if (blocks == 0) blocks = 1;
    note_launch("gemv_q8_vecs", F::TYPE_ID, STEPS, KS, NV, RB, blocks, 1, 256);
    hipLaunchKernelGGL((gemv_q8_vecs<F, STEPS, KS, NV, RB>), dim3(blocks), dim3(256), 0, stream, a.W, a.A, a.a_stride,
                       a.out, a.out_stride, a.n_rows, units, row_bytes, a.accumulate, a.n_vecs, a.bias);
    return hipGetLastError();
}

// Same split of a row over steps and waves as the single-vector kernel (so the fp32 sums are
// formed in the same order and the results are bit-identical to one launch per vector); two
// steps per wave leave registers for two vectors only.
template <class F>
static hipError_t launch_vecs_f(const GemvVecsArgs &a, hipStream_t stream) {
    if (a.n_cols % F::BLOCK_COLS != 0) return hipErrorNotSupported;  // gemv_vecs_max says so beforehand
    const uint32_t units = a.n_cols / F::UNIT_COLS;
    const size_t row_bytes = (size_t)(a.n_cols / F::BLOCK_COLS) * F::BLOCK_BYTES;
    const uint32_t steps = (units + 63) / 64;
    if (steps == 1)
        return a.n_vecs > 2 ? launch_vecs_k<F, 1, 1, 4>(a, units, row_bytes, stream)
                            : launch_vecs_k<F, 1, 1, 2>(a, units, row_bytes, stream);
    if (steps == 2 && a.n_vecs <= 2) return launch_vecs_k<F, 2, 1, 2>(a, units, row_bytes, stream);
    if (steps == 3 || steps == 4)
        return a.n_vecs > 2 ? launch_vecs_k<F, 1, 4, 4>(a, units, row_bytes, stream)
                            : launch_vecs_k<F, 1, 4, 2>(a, units, row_bytes, stream);
    if (steps >= 5 && steps <= 8 && a.n_vecs <= 2) return launch_vecs_k<F, 2, 4, 2>(a, units, row_bytes, stream);
    return hipErrorNotSupported;
}

// One matrix set (GemvArgs::n_mats) of format F: one launch when the register-cached kernel
// takes it, else one launch per matrix.
template <class F>
static hipError_t launch_gemv_format(const GemvArgs &a, uint32_t group_cols, hipStream_t stream) {
    if (a.n_mats > 1 && !multi_in_one_launch<F>(a)) {
        for (uint32_t i = 0; i < a.n_mats; i++) {
            GemvArgs s = a;
            s.n_mats = 1;
            if (i) {
                s.W = a.W_more[i - 1];
                s.out = a.out_more[i - 1];
                s.bias = a.bias_more[i - 1];
                if (a.n_rows_more[i - 1]) s.n_rows = a.n_rows_more[i - 1];
            }
            hipError_t e = launch_format<F>(s, group_cols, stream);
            if (e != hipSuccess) return e;
        }
        return hipSuccess;
    }
    return launch_format<F>(a, group_cols, stream);
}

}  // namespace oxq
