// The GEMV kernels of oxq_gemv.hip instantiated for the formats beyond the first five (Q4_1, Q5_0,
// Q5_1, Q8_1, IQ4_NL, Q2_K, Q3_K, Q5_K): same row streaming, launch policy and multi-matrix /
// multi-vector forms; only the per-format lane work (oxq_formats_more.hpp) differs.  A
// translation unit of its own so that the two sets compile side by side.
#include "oxq_formats_more.hpp"
#include "oxq_gemv_launch.hpp"

namespace oxq {

hipError_t launch_gemv_vecs_more(uint32_t type, const GemvVecsArgs &a, hipStream_t stream) {
    switch (type) {
    case OXQ_TYPE_Q4_1: return launch_vecs_f<FmtQ4_1>(a, stream);
    case OXQ_TYPE_Q5_0: return launch_vecs_f<FmtQ5_0>(a, stream);
    case OXQ_TYPE_Q5_1: return launch_vecs_f<FmtQ5_1>(a, stream);
    case OXQ_TYPE_Q8_1: return launch_vecs_f<FmtQ8_1>(a, stream);
    case OXQ_TYPE_IQ4_NL: return launch_vecs_f<FmtIQ4NL>(a, stream);
    case OXQ_TYPE_Q2_K: return launch_vecs_f<FmtQ2K>(a, stream);
    case OXQ_TYPE_Q3_K: return launch_vecs_f<FmtQ3K>(a, stream);
    case OXQ_TYPE_Q5_K: return launch_vecs_f<FmtQ5K>(a, stream);
    default: return hipErrorInvalidValue;
    }
}

hipError_t launch_gate_up_swiglu_more(uint32_t type, const uint8_t *Wg, const uint8_t *Wu, const uint8_t *acts,
                                      uint8_t *hq, float *h, uint32_t n_rows, uint32_t n_cols, hipStream_t stream,
                                 const GateUpGroups &grp) {
    switch (type) {
    case OXQ_TYPE_Q5_K: return launch_gate_up_swiglu_format<FmtQ5K>(Wg, Wu, acts, hq, h, n_rows, n_cols, stream, grp);
    case OXQ_TYPE_Q4_1: return launch_gate_up_swiglu_format<FmtQ4_1>(Wg, Wu, acts, hq, h, n_rows, n_cols, stream, grp);
    case OXQ_TYPE_Q5_0: return launch_gate_up_swiglu_format<FmtQ5_0>(Wg, Wu, acts, hq, h, n_rows, n_cols, stream, grp);
    case OXQ_TYPE_Q5_1: return launch_gate_up_swiglu_format<FmtQ5_1>(Wg, Wu, acts, hq, h, n_rows, n_cols, stream, grp);
    default: return hipErrorNotSupported;  // the caller runs the two projections and the SwiGLU kernel
    }
}

hipError_t launch_gemv_q8_more(uint32_t type, const GemvArgs &a, hipStream_t stream) {
    switch (type) {
    case OXQ_TYPE_Q4_1: return launch_gemv_format<FmtQ4_1>(a, 32, stream);
    case OXQ_TYPE_Q5_0: return launch_gemv_format<FmtQ5_0>(a, 32, stream);
    case OXQ_TYPE_Q5_1: return launch_gemv_format<FmtQ5_1>(a, 32, stream);
    case OXQ_TYPE_Q8_1: return launch_gemv_format<FmtQ8_1>(a, 32, stream);
    case OXQ_TYPE_IQ4_NL: return launch_gemv_format<FmtIQ4NL>(a, 32, stream);
    case OXQ_TYPE_Q2_K: return launch_gemv_format<FmtQ2K>(a, 16, stream);
    case OXQ_TYPE_Q3_K: return launch_gemv_format<FmtQ3K>(a, 16, stream);
    case OXQ_TYPE_Q5_K: return launch_gemv_format<FmtQ5K>(a, 32, stream);
    default: return hipErrorInvalidValue;
    }
}

}  // namespace oxq
