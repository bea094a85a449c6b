// Batched (prefill) form of the fused matvec: out[m x n] (+)= A_q8[m rows] x W[n x k]^T.
#include "oxq_formats.hpp"
#include "oxq_internal.hpp"

namespace oxq {

// One fused matvec per activation row (what every gemm of the reference does,
// crates/oxillama-quant/src/reference/q4_k.rs:186-201).
static hipError_t gemm_by_rows(uint32_t type, const GemmArgs &a, hipStream_t stream) {
    const size_t act_row_bytes = (size_t)(a.k / 32) * 34;
    for (uint32_t r = 0; r < a.m; r++) {
        GemvArgs g;
        g.W = a.W;
        g.A = a.A + r * act_row_bytes;
        g.out = a.out + (size_t)r * a.n;
        g.sums = nullptr;
        g.n_rows = a.n;
        g.n_cols = a.k;
        g.accumulate = a.accumulate;
        g.waves_per_cu = 8;
        g.rows_per_batch = 0;
        g.waves_per_row = 0;
        hipError_t e = launch_gemv_q8(type, g, stream);
        if (e != hipSuccess) return e;
    }
    return hipSuccess;
}

hipError_t launch_gemm_q8(uint32_t type, const GemmArgs &a, hipStream_t stream) {
    return gemm_by_rows(type, a, stream);
}

}  // namespace oxq
