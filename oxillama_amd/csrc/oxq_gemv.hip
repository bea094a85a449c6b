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
#include "oxq_gemv_launch.hpp"

namespace oxq {

// Columns of a lane's unit, by format (0: unknown type).
uint32_t gemv_unit_cols(uint32_t type) {
    switch (type) {
    case OXQ_TYPE_Q4_K:
    case OXQ_TYPE_Q6_K:
    case OXQ_TYPE_Q5_K:
    case OXQ_TYPE_Q2_K:
    case OXQ_TYPE_Q3_K: return 64;
    case OXQ_TYPE_Q4_0:
    case OXQ_TYPE_Q8_0:
    case OXQ_TYPE_IQ4_XS:
    case OXQ_TYPE_Q4_1:
    case OXQ_TYPE_Q5_0:
    case OXQ_TYPE_Q5_1:
    case OXQ_TYPE_Q8_1:
    case OXQ_TYPE_IQ4_NL: return 32;
    default: return 0;
    }
}

// Weights per exact integer group sum (the debug dump's granularity).
uint32_t gemv_group_cols(uint32_t type) {
    return type == OXQ_TYPE_Q6_K || type == OXQ_TYPE_Q2_K || type == OXQ_TYPE_Q3_K ? 16 : 32;
}

// Most activation vectors one launch takes for rows of n_cols columns (0: none).
uint32_t gemv_vecs_max(uint32_t type, uint32_t n_cols) {
    const uint32_t unit = gemv_unit_cols(type);
    if (unit == 0) return 0;
    if (n_cols % (uint32_t)oxq_block_size(type) != 0) return 0;  // rows that end inside a block: one vector per launch
    const uint32_t steps = (n_cols / unit + 63) / 64;
    if (steps == 1 || steps == 3 || steps == 4) return 4;
    if (steps == 2 || (steps >= 5 && steps <= 8)) return 2;
    return 0;
}

// The Q6_K lane policy loads from the dword-aligned address at or below its bytes, which for the first
// block of a matrix must not lie before the matrix.
static bool misaligned(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 3) != 0; }

// 2..4 activation vectors (3 run in the 4-vector kernel, which repeats the last one).
hipError_t launch_gemv_vecs(uint32_t type, const GemvVecsArgs &a, hipStream_t stream) {
    if (a.n_rows == 0 || a.n_cols == 0) return hipSuccess;
    switch (type) {
    case OXQ_TYPE_Q4_0: return launch_vecs_f<FmtQ4_0>(a, stream);
    case OXQ_TYPE_Q8_0: return launch_vecs_f<FmtQ8_0>(a, stream);
    case OXQ_TYPE_Q4_K: return launch_vecs_f<FmtQ4K>(a, stream);
    case OXQ_TYPE_Q6_K: return misaligned(a.W) ? hipErrorInvalidDevicePointer : launch_vecs_f<FmtQ6K>(a, stream);
    case OXQ_TYPE_IQ4_XS: return launch_vecs_f<FmtIQ4XS>(a, stream);
    default: return launch_gemv_vecs_more(type, a, stream);
    }
}

bool gemv_takes_f32(uint32_t type, uint32_t n_cols) {
    const uint32_t unit = gemv_unit_cols(type);
    // the register-cached kernel (up to 8 steps, or 4 waves x 8) and the default dynamic LDS limit
    if (unit == 0) return false;
    const uint32_t bs = (uint32_t)oxq_block_size(type), units = (n_cols + bs - 1) / bs * (bs / unit);
    return (units + 63) / 64 <= 32 && (size_t)units * (unit / 32) * 34 <= 48 * 1024;
}

hipError_t launch_gate_up_swiglu(uint32_t type, const uint8_t *Wg, const uint8_t *Wu, const uint8_t *acts, uint8_t *hq,
                                 float *h, uint32_t n_rows, uint32_t n_cols, hipStream_t stream,
                                 const GateUpGroups &grp) {
    switch (type) {
    case OXQ_TYPE_Q4_0: return launch_gate_up_swiglu_format<FmtQ4_0>(Wg, Wu, acts, hq, h, n_rows, n_cols, stream, grp);
    case OXQ_TYPE_Q8_0: return launch_gate_up_swiglu_format<FmtQ8_0>(Wg, Wu, acts, hq, h, n_rows, n_cols, stream, grp);
    case OXQ_TYPE_Q4_K: return launch_gate_up_swiglu_format<FmtQ4K>(Wg, Wu, acts, hq, h, n_rows, n_cols, stream, grp);
    case OXQ_TYPE_Q6_K:
        if (misaligned(Wg) || misaligned(Wu)) return hipErrorInvalidDevicePointer;
        return launch_gate_up_swiglu_format<FmtQ6K>(Wg, Wu, acts, hq, h, n_rows, n_cols, stream, grp);
    case OXQ_TYPE_IQ4_XS: return launch_gate_up_swiglu_format<FmtIQ4XS>(Wg, Wu, acts, hq, h, n_rows, n_cols, stream, grp);
    default: return launch_gate_up_swiglu_more(type, Wg, Wu, acts, hq, h, n_rows, n_cols, stream, grp);
    }
}

hipError_t launch_gemv_q8(uint32_t type, const GemvArgs &a, hipStream_t stream) {
    if (a.n_rows == 0 || a.n_cols == 0) return hipSuccess;
    switch (type) {
    case OXQ_TYPE_Q4_0: return launch_gemv_format<FmtQ4_0>(a, 32, stream);
    case OXQ_TYPE_Q8_0: return launch_gemv_format<FmtQ8_0>(a, 32, stream);
    case OXQ_TYPE_Q4_K: return launch_gemv_format<FmtQ4K>(a, 32, stream);
    case OXQ_TYPE_Q6_K:
        if (misaligned(a.W)) return hipErrorInvalidDevicePointer;
        for (uint32_t i = 1; i < a.n_mats; i++)
            if (misaligned(a.W_more[i - 1])) return hipErrorInvalidDevicePointer;
        return launch_gemv_format<FmtQ6K>(a, 16, stream);
    case OXQ_TYPE_IQ4_XS: return launch_gemv_format<FmtIQ4XS>(a, 32, stream);
    default: return launch_gemv_q8_more(type, a, stream);
    }
}

}  // namespace oxq
