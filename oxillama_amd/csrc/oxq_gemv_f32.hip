// QuantKernel::gemv with the reference's own numerics (gfx950): fp32 activations against weights
// dequantized in registers, every term formed as the reference's scalar rows form it
// (crates/oxillama-quant/src/reference/q4_0.rs:82-102, q8_0.rs:77-92, q4_k.rs:135-178, q6_k.rs:108-166,
// iq4_xs.rs:130-163).  The Q8_0-activation kernels (oxq_gemv.hip) quantize x first, which is the reference's
// matvec_q8_fused, not its gemv; this file is the route for callers that want gemv's result.
//
// Work split as in the Q8_0-activation kernel: lane l of a wave owns unit 64 s + l of a row (the same units, so
// the weight loads are the format policies' load_w), KS waves share a row, rows are dealt round-robin to wave
// groups, the next row's weights are requested before this row's are used.  A lane keeps the activations of its
// units in registers for all rows (32 or 64 floats per unit).  Inside a unit the terms are added in the
// reference's column order with its expression (no contraction: the file is compiled with -ffp-contract=off);
// across units the reference's running sum becomes a tree (lanes, then waves in order), which moves the result by
// rounding only: |y - y_ref| stays far inside 1e-5 |y|inf (tests/test_gpu_gemv_f32.py).
#include "oxq_formats.hpp"
#include "oxq_internal.hpp"

namespace oxq {

// ---- per-format: which columns a unit covers, and its contribution --------------------------------------------
// load_x: the lane's activations for unit u, in the order dot() uses them; columns >= n_cols read as 0.0f (the
// reference skips them; a zero factor adds a zero term).

__device__ __forceinline__ void load_x_run(float *dst, const float *__restrict__ x, uint32_t col, uint32_t count,
                                           uint32_t n_cols) {
    for (uint32_t i = 0; i < count; i += 4) {
        if (col + i + 4 <= n_cols) {
            const u32x4 raw = ld16(reinterpret_cast<const uint8_t *>(x + col + i));
            for (int j = 0; j < 4; j++) {
                const uint32_t bits = raw[j];
                dst[i + j] = __builtin_bit_cast(float, bits);
            }
        } else {
            for (int j = 0; j < 4; j++) dst[i + j] = col + i + j < n_cols ? x[col + i + j] : 0.0f;
        }
    }
}

template <class F>
struct F32Dot {
    static constexpr bool OK = false;
};

template <>
struct F32Dot<FmtQ8_0> {
    static constexpr bool OK = true;
    static __device__ __forceinline__ void load_x(float (&xs)[32], const float *x, uint32_t u, uint32_t n_cols,
                                                  const FmtQ8_0::Lane &) {
        load_x_run(xs, x, 32 * u, 32, n_cols);
    }
    static __device__ __forceinline__ float dot(const FmtQ8_0::Wt &w, const float (&xs)[32], const FmtQ8_0::Lane &) {
        const uint32_t sh = w.off ? 0u : 16u;
        const uint32_t dw[9] = {w.q0[0], w.q0[1], w.q0[2], w.q0[3], w.q1[0], w.q1[1], w.q1[2], w.q1[3], w.x};
        const float d = h2f(w.off ? w.x : (w.q0[0] & 0xFFFFu));
        float sum = 0.0f;
        for (int i = 0; i < 8; i++) {
            const uint32_t q = __builtin_amdgcn_alignbit(dw[i + 1], dw[i], sh);
            for (int b = 0; b < 4; b++)  // q8_0.rs:88: sum += q as f32 * d * x
                sum += (float)(int8_t)(q >> (8 * b)) * d * xs[4 * i + b];
        }
        return sum;
    }
};

template <>
struct F32Dot<FmtQ4_0> {
    static constexpr bool OK = true;
    static __device__ __forceinline__ void load_x(float (&xs)[32], const float *x, uint32_t u, uint32_t n_cols,
                                                  const FmtQ4_0::Lane &) {
        load_x_run(xs, x, 32 * u, 32, n_cols);
    }
    static __device__ __forceinline__ float dot(const FmtQ4_0::Wt &w, const float (&xs)[32], const FmtQ4_0::Lane &) {
        const uint32_t sh = w.off ? 0u : 16u;
        const uint32_t dw[5] = {w.q[0], w.q[1], w.q[2], w.q[3], w.x};
        const float d = h2f(w.off ? w.x : (w.q[0] & 0xFFFFu));
        float sum = 0.0f;
        for (int i = 0; i < 4; i++) {
            const uint32_t q = __builtin_amdgcn_alignbit(dw[i + 1], dw[i], sh);
            for (int b = 0; b < 4; b++) {  // q4_0.rs:93-98: byte j -> columns 2j (low nibble), 2j + 1 (high)
                const uint32_t byte = (q >> (8 * b)) & 0xFFu;
                const int lo = (int)(byte & 0x0Fu) - 8, hi = (int)(byte >> 4) - 8;
                sum += (float)lo * d * xs[8 * i + 2 * b];
                sum += (float)hi * d * xs[8 * i + 2 * b + 1];
            }
        }
        return sum;
    }
};

template <>
struct F32Dot<FmtQ4K> {
    static constexpr bool OK = true;
    static __device__ __forceinline__ void load_x(float (&xs)[64], const float *x, uint32_t u, uint32_t n_cols,
                                                  const FmtQ4K::Lane &k) {
        load_x_run(xs, x, 256 * (u >> 2) + 64 * k.g, 64, n_cols);
    }
    static __device__ __forceinline__ float dot(const FmtQ4K::Wt &w, const float (&xs)[64], const FmtQ4K::Lane &k) {
        // scales / mins of sub-blocks 2g, 2g + 1 (decode_scales_mins, q4_k.rs:27-49), as in FmtQ4K::dot
        const uint32_t sa = w.hdr[1] >> k.sh, sb = w.hdr[2] >> k.sh, sc3 = w.hdr[3] >> k.sh;
        const uint32_t xx = k.upper ? sc3 : sa, yy = k.upper ? (sc3 >> 4) : sb;
        const uint32_t m1 = k.upper ? 0x0F0Fu : 0x3F3Fu, m2 = k.upper ? 0x3030u : 0u;
        const uint32_t sc2 = (xx & m1) | ((sa >> 2) & m2);
        const uint32_t mn2 = (yy & m1) | ((sb >> 2) & m2);
        const float d = h2f(w.hdr[0] & 0xFFFF), dmin = h2f(w.hdr[0] >> 16);
        const float d1 = d * (float)(sc2 & 0xFF), mm1 = dmin * (float)(mn2 & 0xFF);                // q4_k.rs:151-152
        const float d2 = d * (float)((sc2 >> 8) & 0xFF), mm2 = dmin * (float)((mn2 >> 8) & 0xFF);  // q4_k.rs:153-154
        const uint32_t qs[8] = {w.q0[0], w.q0[1], w.q0[2], w.q0[3], w.q1[0], w.q1[1], w.q1[2], w.q1[3]};
        float sum = 0.0f;
        for (int l = 0; l < 32; l++) {  // q4_k.rs:157-163
            const float q = (float)((qs[l >> 2] >> (8 * (l & 3))) & 0x0Fu);
            sum += (d1 * q - mm1) * xs[l];
        }
        for (int l = 0; l < 32; l++) {  // q4_k.rs:164-170
            const float q = (float)((qs[l >> 2] >> (8 * (l & 3) + 4)) & 0x0Fu);
            sum += (d2 * q - mm2) * xs[32 + l];
        }
        return sum;
    }
};

template <>
struct F32Dot<FmtQ6K> {
    static constexpr bool OK = true;
    // unit (block b, half hh, sixteen is): columns 256 b + 128 hh + 32 j + 16 is + t, j = 0..3, t = 0..15
    static __device__ __forceinline__ void load_x(float (&xs)[64], const float *x, uint32_t u, uint32_t n_cols,
                                                  const FmtQ6K::Lane &k) {
        for (int j = 0; j < 4; j++)
            load_x_run(xs + 16 * j, x, 256 * (u >> 2) + 128 * k.hh + 32 * j + 16 * k.is, 16, n_cols);
    }
    static __device__ __forceinline__ float dot(const FmtQ6K::Wt &w, const float (&xs)[64], const FmtQ6K::Lane &k) {
        // the lane's bytes, put in place as FmtQ6K::dot does (loads come from the dword-aligned address below)
        const uint32_t x_ql0 = FmtQ6K::qp<0xB1>(w.ql0[0]), x_ql1 = FmtQ6K::qp<0xB1>(w.ql1[0]),
                       x_qh = FmtQ6K::qp<0xB1>(w.qh[0]);
        const uint32_t p2_ql0 = FmtQ6K::qp<0xAA>(w.ql0[0]), p2_qh = FmtQ6K::qp<0xAA>(w.qh[0]);
        const uint32_t p0_qh = FmtQ6K::qp<0x00>(w.qh[0]), p0_sc = FmtQ6K::qp<0x00>(w.sc[0]);
        const u32x4 ql0 = FmtQ6K::realign(w.ql0, k.is ? x_ql1 : x_ql0, w.sh);
        const u32x4 ql1 = FmtQ6K::realign(w.ql1, k.is ? (k.hh ? p0_qh : p2_ql0) : x_ql1, w.sh);
        const u32x4 qh = FmtQ6K::realign(w.qh, k.is ? (k.hh ? p0_sc : p2_qh) : x_qh, w.sh);
        const uint32_t s0 = __builtin_amdgcn_alignbit(w.sc[1], w.sc[0], w.sh) >> (8 * k.is);
        const uint32_t s1 = __builtin_amdgcn_alignbit(w.sc2, w.sc[1], w.sh) >> (8 * k.is);
        const float d = h2f(w.d);
        // q6_k.rs:131-134: s_j = d * scales[8 hh + is + 2 j]
        const float sj[4] = {d * (float)(int8_t)(s0 & 0xFF), d * (float)(int8_t)((s0 >> 16) & 0xFF),
                             d * (float)(int8_t)(s1 & 0xFF), d * (float)(int8_t)((s1 >> 16) & 0xFF)};
        float sum = 0.0f;
        for (int t = 0; t < 16; t++) {  // q6_k.rs:124-160: l = 16 is + t, the four quarters of the half in turn
            const uint32_t sh8 = 8 * (t & 3);
            const uint32_t l0 = (ql0[t >> 2] >> sh8) & 0xFFu, l1 = (ql1[t >> 2] >> sh8) & 0xFFu,
                           h = (qh[t >> 2] >> sh8) & 0xFFu;
            const int q0 = (int)((l0 & 0x0F) | ((h & 3) << 4)) - 32;         // q6_k.rs:55
            const int q1 = (int)((l1 & 0x0F) | (((h >> 2) & 3) << 4)) - 32;  // q6_k.rs:56
            const int q2 = (int)((l0 >> 4) | (((h >> 4) & 3) << 4)) - 32;    // q6_k.rs:57
            const int q3 = (int)((l1 >> 4) | (((h >> 6) & 3) << 4)) - 32;    // q6_k.rs:58
            sum += sj[0] * (float)q0 * xs[t];
            sum += sj[1] * (float)q1 * xs[16 + t];
            sum += sj[2] * (float)q2 * xs[32 + t];
            sum += sj[3] * (float)q3 * xs[48 + t];
        }
        return sum;
    }
};

template <>
struct F32Dot<FmtIQ4XS> {
    static constexpr bool OK = true;
    static __device__ __forceinline__ void load_x(float (&xs)[32], const float *x, uint32_t u, uint32_t n_cols,
                                                  const FmtIQ4XS::Lane &) {
        load_x_run(xs, x, 32 * u, 32, n_cols);
    }
    static __device__ __forceinline__ float dot(const FmtIQ4XS::Wt &w, const float (&xs)[32], const FmtIQ4XS::Lane &k) {
        const uint32_t ls_low = (w.hdr[1] >> (4 * k.i)) & 0x0F;
        const uint32_t ls_high = ((w.hdr[0] >> 16) >> (2 * k.i)) & 0x03;
        const int ls = (int)(ls_low | (ls_high << 4)) - 32;       // unpack_sub_scale, iq4_xs.rs:47-53
        const float scale = h2f(w.hdr[0] & 0xFFFF) * (float)ls;  // iq4_xs.rs:145
        float sum = 0.0f;
        for (int i = 0; i < 4; i++) {
            const uint32_t lo = FmtIQ4XS::lut4(w.q[i] & 0x0F0F0F0Fu), hi = FmtIQ4XS::lut4((w.q[i] >> 4) & 0x0F0F0F0Fu);
            for (int b = 0; b < 4; b++) {  // iq4_xs.rs:148-157: byte j -> columns 2j, 2j + 1
                sum += (float)(int8_t)(lo >> (8 * b)) * scale * xs[8 * i + 2 * b];
                sum += (float)(int8_t)(hi >> (8 * b)) * scale * xs[8 * i + 2 * b + 1];
            }
        }
        return sum;
    }
};

// ---- kernel --------------------------------------------------------------------------------------------------

template <class F, int STEPS, int KS>
__global__ __launch_bounds__(256) void gemv_f32_kernel(const uint8_t *__restrict__ W, const float *__restrict__ x,
                                                      float *__restrict__ out, const float *__restrict__ old,
                                                      uint32_t n_rows, uint32_t units, size_t row_bytes,
                                                      uint32_t n_cols) {
    constexpr uint32_t G = 4 / KS, UC = F::UNIT_COLS;
    __shared__ float part_sums[2][4];
    const uint32_t lane = threadIdx.x & 63;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const uint32_t part = wave % KS, grp = wave / KS;
    const uint32_t group = blockIdx.x * G + grp, n_groups = gridDim.x * G;
    const uint32_t unit0 = part * STEPS * 64;
    const typename F::Lane k = F::lane_consts(lane);
    // with KS > 1 every wave of a work group makes the same number of trips (barriers)
    const uint32_t n_trips = KS == 1 ? n_rows : ((n_rows + n_groups - 1) / n_groups) * n_groups;
    if (KS == 1 && group >= n_rows) return;

    auto load_row = [&](typename F::Wt (&w)[STEPS], uint32_t row) {
        const uint8_t *rp = W + (size_t)min(row, n_rows - 1) * row_bytes;  // past the end: the last row, unused
#pragma unroll
        for (int s = 0; s < STEPS; s++) F::load_w(w[s], rp, min(unit0 + (uint32_t)(s * 64) + lane, units - 1), k);
    };
    typename F::Wt w0[STEPS], w1[STEPS];
    load_row(w0, group);
    float xs[STEPS][UC];
#pragma unroll
    for (int s = 0; s < STEPS; s++) {
        const uint32_t u = unit0 + (uint32_t)(s * 64) + lane;
        // a unit past the end of the row: activations 0, weights those of the last unit
        F32Dot<F>::load_x(xs[s], x, min(u, units - 1), u < units ? n_cols : 0u, k);
    }
    uint32_t trip = 0;
    auto finish = [&](const typename F::Wt (&w)[STEPS], uint32_t row) {
        float acc = 0.0f;
#pragma unroll
        for (int s = 0; s < STEPS; s++) acc += F32Dot<F>::dot(w[s], xs[s], k);
        const float total = wave_sum(acc);
        if (KS == 1) {
            if (lane == 0 && row < n_rows) out[row] = old ? old[row] + total : total;
        } else {
            if (lane == 0) part_sums[trip & 1][wave] = total;
            __syncthreads();
            if (part == 0 && lane == 0 && row < n_rows) {
                float t = part_sums[trip & 1][grp * KS];
#pragma unroll
                for (int p = 1; p < KS; p++) t += part_sums[trip & 1][grp * KS + p];
                out[row] = old ? old[row] + t : t;
            }
            trip++;
        }
    };
    uint32_t row = group;
    while (true) {
        const uint32_t next = row + n_groups;
        if (next >= n_trips) {
            finish(w0, row);
            break;
        }
        load_row(w1, next);
        finish(w0, row);
        const uint32_t next2 = next + n_groups;
        if (next2 >= n_trips) {
            finish(w1, next);
            break;
        }
        load_row(w0, next2);
        finish(w1, next);
        row = next2;
    }
}

// Rows longer than the register kernel takes: one wave per row walks the units 64 at a time and reads the
// activations again for every row (from L2).
template <class F>
__global__ __launch_bounds__(256) void gemv_f32_long(const uint8_t *__restrict__ W, const float *__restrict__ x,
                                                    float *__restrict__ out, const float *__restrict__ old,
                                                    uint32_t n_rows, uint32_t units, size_t row_bytes, uint32_t n_cols) {
    const uint32_t lane = threadIdx.x & 63;
    const uint32_t wave = blockIdx.x * 4 + (threadIdx.x >> 6), n_waves = gridDim.x * 4;
    const typename F::Lane k = F::lane_consts(lane);
    for (uint32_t row = wave; row < n_rows; row += n_waves) {
        const uint8_t *rp = W + (size_t)row * row_bytes;
        float acc = 0.0f;
        for (uint32_t u0 = 0; u0 < units; u0 += 64) {
            const uint32_t u = u0 + lane;
            typename F::Wt w;
            float xs[F::UNIT_COLS];
            F::load_w(w, rp, min(u, units - 1), k);
            F32Dot<F>::load_x(xs, x, min(u, units - 1), u < units ? n_cols : 0u, k);
            acc += F32Dot<F>::dot(w, xs, k);
        }
        const float total = wave_sum(acc);
        if (lane == 0) out[row] = old ? old[row] + total : total;
    }
}

template <class F, int STEPS, int KS>
static hipError_t launch_f32_k(const uint8_t *W, const float *x, float *out, const float *old, uint32_t n_rows,
                               uint32_t units, size_t row_bytes, uint32_t n_cols, hipStream_t stream) {
    constexpr uint32_t G = 4 / KS;
    const uint32_t max_groups = device_cus() * 8 / KS;  // eight waves per compute unit
    const uint32_t passes = (n_rows + max_groups - 1) / max_groups;
    const uint32_t groups = (n_rows + passes - 1) / passes;
    const uint32_t blocks = (groups + G - 1) / G;
    note_launch("gemv_f32", F::TYPE_ID, STEPS, KS, 0, 0, blocks, 1, 256);
    hipLaunchKernelGGL((gemv_f32_kernel<F, STEPS, KS>), dim3(blocks ? blocks : 1), dim3(256), 0, stream, W, x, out, old,
                       n_rows, units, row_bytes, n_cols);
    return hipGetLastError();
}

template <class F>
static hipError_t launch_f32_format(const uint8_t *W, const float *x, float *out, const float *old, uint32_t n_rows,
                                    uint32_t n_cols, hipStream_t stream) {
    const uint32_t blocks_per_row = (n_cols + F::BLOCK_COLS - 1) / F::BLOCK_COLS;
    const uint32_t units = blocks_per_row * (F::BLOCK_COLS / F::UNIT_COLS);
    const size_t row_bytes = (size_t)blocks_per_row * F::BLOCK_BYTES;
    const uint32_t steps = (units + 63) / 64;
    // a lane holds UNIT_COLS floats per step: one step of a 64-column unit, two of a 32-column one
    constexpr uint32_t MAX_STEPS = 64 / F::UNIT_COLS;
    if (steps <= 1) return launch_f32_k<F, 1, 1>(W, x, out, old, n_rows, units, row_bytes, n_cols, stream);
    if constexpr (MAX_STEPS >= 2) {
        if (steps == 2) return launch_f32_k<F, 2, 1>(W, x, out, old, n_rows, units, row_bytes, n_cols, stream);
    }
    if (steps <= 4) return launch_f32_k<F, 1, 4>(W, x, out, old, n_rows, units, row_bytes, n_cols, stream);
    if constexpr (MAX_STEPS >= 2) {
        if (steps <= 8) return launch_f32_k<F, 2, 4>(W, x, out, old, n_rows, units, row_bytes, n_cols, stream);
    }
    const uint32_t waves = min(n_rows, device_cus() * 8);
    note_launch("gemv_f32_long", F::TYPE_ID, 0, 0, 0, 0, (waves + 3) / 4, 1, 256);
    hipLaunchKernelGGL((gemv_f32_long<F>), dim3((waves + 3) / 4), dim3(256), 0, stream, W, x, out, old, n_rows, units,
                       row_bytes, n_cols);
    return hipGetLastError();
}

bool gemv_f32_supported(uint32_t type) {
    return type == OXQ_TYPE_Q4_0 || type == OXQ_TYPE_Q8_0 || type == OXQ_TYPE_Q4_K || type == OXQ_TYPE_Q6_K ||
           type == OXQ_TYPE_IQ4_XS;
}

// out[r] = (old ? old[r] : 0) + W[r, :] . x with the reference gemv's per-term arithmetic.
hipError_t launch_gemv_f32(uint32_t type, const uint8_t *W, const float *x, float *out, const float *old,
                           uint32_t n_rows, uint32_t n_cols, hipStream_t stream) {
    if (n_rows == 0 || n_cols == 0) return hipSuccess;
    switch (type) {
    case OXQ_TYPE_Q4_0: return launch_f32_format<FmtQ4_0>(W, x, out, old, n_rows, n_cols, stream);
    case OXQ_TYPE_Q8_0: return launch_f32_format<FmtQ8_0>(W, x, out, old, n_rows, n_cols, stream);
    case OXQ_TYPE_Q4_K: return launch_f32_format<FmtQ4K>(W, x, out, old, n_rows, n_cols, stream);
    case OXQ_TYPE_Q6_K:
        if ((reinterpret_cast<uintptr_t>(W) & 3) != 0) return hipErrorInvalidDevicePointer;  // FmtQ6K::load_w
        return launch_f32_format<FmtQ6K>(W, x, out, old, n_rows, n_cols, stream);
    case OXQ_TYPE_IQ4_XS: return launch_f32_format<FmtIQ4XS>(W, x, out, old, n_rows, n_cols, stream);
    default: return hipErrorNotSupported;
    }
}

}  // namespace oxq
