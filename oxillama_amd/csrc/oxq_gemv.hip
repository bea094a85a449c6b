// Batch-1 fused GEMV over raw GGUF blocks with Q8_0 activations (gfx950).
//
// One wave owns whole rows: lane l handles units 64*s + l of the row for every
// step s.  The activation bytes a lane needs do not depend on the row, so they
// are loaded once into registers; per row the wave then only streams weight
// bytes (coalesced 16-byte loads of the untouched GGUF blocks), forms exact
// int32 group sums with v_dot4 and one fp32 term per group, and reduces across
// the wave with DPP.  No MFMA: the kernel is bound by HBM, not by arithmetic.
//
// Replaces the row loops of QuantKernel::matvec_q8_fused in the reference
// (crates/oxillama-quant/src/traits.rs:89-173, reference/q4_k.rs:218-333,
// reference/q6_k.rs:212-354, simd/avx2/{q4_0,q8_0,q4_k,q6_k}.rs).
#include "oxq_formats.hpp"
#include "oxq_internal.hpp"

namespace oxq {

// STEPS > 0: activations for all steps cached in registers, RB rows in flight.
template <class F, int STEPS, int RB, bool DUMP>
__global__ __launch_bounds__(256) void gemv_q8_cached(const uint8_t *__restrict__ W,
                                                     const uint8_t *__restrict__ A,
                                                     float *__restrict__ out, int32_t *__restrict__ sums,
                                                     uint32_t n_rows, uint32_t units, uint32_t groups_per_row,
                                                     size_t row_bytes, int accumulate) {
    const uint32_t lane = threadIdx.x & 63;
    const uint32_t wave = __builtin_amdgcn_readfirstlane((blockIdx.x * blockDim.x + threadIdx.x) >> 6);
    const uint32_t n_waves = (gridDim.x * blockDim.x) >> 6;
    const typename F::Lane k = F::lane_consts(lane);

    typename F::Act act[STEPS];
    bool valid[STEPS];
#pragma unroll
    for (int s = 0; s < STEPS; s++) {
        const uint32_t u = s * 64 + lane;
        valid[s] = u < units;
        F::load_act(act[s], A, u, valid[s], k);
    }

    const uint32_t n_batches = (n_rows + RB - 1) / RB;
    for (uint32_t batch = wave; batch < n_batches; batch += n_waves) {
        const uint32_t row0 = batch * RB;
        typename F::Wt w[RB][STEPS];
        float old = 0.0f;
        if (accumulate && lane < RB && row0 + lane < n_rows) old = out[row0 + lane];
#pragma unroll
        for (int r = 0; r < RB; r++) {
            const uint32_t row = min(row0 + r, n_rows - 1);
            const uint8_t *rp = W + (size_t)row * row_bytes;
#pragma unroll
            for (int s = 0; s < STEPS; s++) F::load_w(w[r][s], rp, s * 64 + lane, valid[s], k);
        }
        float res = 0.0f;
#pragma unroll
        for (int r = 0; r < RB; r++) {
            const uint32_t row = min(row0 + r, n_rows - 1);
            float acc = 0.0f;
#pragma unroll
            for (int s = 0; s < STEPS; s++)
                acc += F::template dot<DUMP>(w[r][s], act[s], k, DUMP ? sums + (size_t)row * groups_per_row : nullptr,
                                             s * 64 + lane, valid[s]);
            const float total = wave_sum(acc);
            if (lane == (uint32_t)r) res = total;
        }
        if (lane < RB && row0 + lane < n_rows) out[row0 + lane] = old + res;
    }
}

// Any number of steps: activations re-read (from L2) for every row.
template <class F, bool DUMP>
__global__ __launch_bounds__(256) void gemv_q8_generic(const uint8_t *__restrict__ W,
                                                      const uint8_t *__restrict__ A,
                                                      float *__restrict__ out, int32_t *__restrict__ sums,
                                                      uint32_t n_rows, uint32_t units, uint32_t groups_per_row,
                                                      size_t row_bytes, int accumulate) {
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
            F::load_w(w, rp, u, valid, k);
            F::load_act(a, A, u, valid, k);
            acc += F::template dot<DUMP>(w, a, k, DUMP ? sums + (size_t)row * groups_per_row : nullptr, u, valid);
        }
        const float total = wave_sum(acc);
        if (lane == 0) out[row] = (accumulate ? out[row] : 0.0f) + total;
    }
}

template <class F, int STEPS, int RB>
static hipError_t launch_cached(const GemvArgs &a, uint32_t units, uint32_t groups_per_row, size_t row_bytes,
                                hipStream_t stream) {
    const uint32_t n_batches = (a.n_rows + RB - 1) / RB;
    const uint32_t max_waves = device_cus() * a.waves_per_cu;
    uint32_t waves = n_batches < max_waves ? n_batches : max_waves;
    uint32_t blocks = (waves + 3) / 4;
    if (blocks == 0) blocks = 1;
    if (a.sums)
        hipLaunchKernelGGL((gemv_q8_cached<F, STEPS, RB, true>), dim3(blocks), dim3(256), 0, stream, a.W, a.A, a.out,
                           a.sums, a.n_rows, units, groups_per_row, row_bytes, a.accumulate);
    else
        hipLaunchKernelGGL((gemv_q8_cached<F, STEPS, RB, false>), dim3(blocks), dim3(256), 0, stream, a.W, a.A,
                           a.out, a.sums, a.n_rows, units, groups_per_row, row_bytes, a.accumulate);
    return hipGetLastError();
}

template <class F>
static hipError_t launch_format(const GemvArgs &a, uint32_t group_cols, hipStream_t stream) {
    const uint32_t units = a.n_cols / F::UNIT_COLS;
    const uint32_t groups_per_row = a.n_cols / group_cols;
    const size_t row_bytes = (size_t)(a.n_cols / F::BLOCK_COLS) * F::BLOCK_BYTES;
    const uint32_t steps = (units + 63) / 64;
    switch (steps) {
    case 1: return launch_cached<F, 1, 4>(a, units, groups_per_row, row_bytes, stream);
    case 2: return launch_cached<F, 2, 4>(a, units, groups_per_row, row_bytes, stream);
    case 3: return launch_cached<F, 3, 2>(a, units, groups_per_row, row_bytes, stream);
    case 4: return launch_cached<F, 4, 2>(a, units, groups_per_row, row_bytes, stream);
    case 5:
    case 6:
    case 7:
    case 8: return launch_cached<F, 8, 1>(a, units, groups_per_row, row_bytes, stream);
    default: break;
    }
    const uint32_t max_waves = device_cus() * a.waves_per_cu;
    uint32_t waves = a.n_rows < max_waves ? a.n_rows : max_waves;
    uint32_t blocks = (waves + 3) / 4;
    if (blocks == 0) blocks = 1;
    if (a.sums)
        hipLaunchKernelGGL((gemv_q8_generic<F, true>), dim3(blocks), dim3(256), 0, stream, a.W, a.A, a.out, a.sums,
                           a.n_rows, units, groups_per_row, row_bytes, a.accumulate);
    else
        hipLaunchKernelGGL((gemv_q8_generic<F, false>), dim3(blocks), dim3(256), 0, stream, a.W, a.A, a.out, a.sums,
                           a.n_rows, units, groups_per_row, row_bytes, a.accumulate);
    return hipGetLastError();
}

hipError_t launch_gemv_q8(uint32_t type, const GemvArgs &a, hipStream_t stream) {
    if (a.n_rows == 0 || a.n_cols == 0) return hipSuccess;
    switch (type) {
    case OXQ_TYPE_Q4_0: return launch_format<FmtQ4_0>(a, 32, stream);
    case OXQ_TYPE_Q8_0: return launch_format<FmtQ8_0>(a, 32, stream);
    case OXQ_TYPE_Q4_K: return launch_format<FmtQ4K>(a, 32, stream);
    case OXQ_TYPE_Q6_K: return launch_format<FmtQ6K>(a, 16, stream);
    case OXQ_TYPE_IQ4_XS: return launch_format<FmtIQ4XS>(a, 32, stream);
    default: return hipErrorInvalidValue;
    }
}

}  // namespace oxq
