// Q8_0 activation quantizer and block dequantizer (gfx950).
//
// quantize: bit-exact twin of encode_q8_0_block in the reference
// (crates/oxillama-quant/src/quantize.rs:190-210): amax over 32 floats, d =
// amax/127, id = 1/d (0 when d == 0), q = clamp(round_half_away(x*id)), d stored
// as f16 (round to nearest even).  Quantisation uses the unrounded fp32 id.
//
// dequant: element-wise restatement of the reference's dequant_block methods
// (reference/{q4_0,q8_0,q4_k,q6_k,iq4_xs}.rs), same fp32 operation order.
#include "oxq_device.hpp"
#include "oxq_internal.hpp"
#include "oxq_q8_encode.hpp"

namespace oxq {

// Eight lanes per 32-float block, four floats per lane.
__global__ __launch_bounds__(256) void quantize_q8_0_kernel(const float *__restrict__ x,
                                                           uint8_t *__restrict__ out, size_t n_blocks) {
    const size_t t = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const size_t blk = t >> 3;
    const uint32_t j = (uint32_t)(t & 7);
    const bool valid = blk < n_blocks;
    float v[4] = {0.0f, 0.0f, 0.0f, 0.0f};
    if (valid) load4(v, x + blk * 32 + 4 * j);
    encode_q8_0_lanes(v, valid, out + blk * 34, j);
}

hipError_t launch_quantize_q8_0(const float *x, size_t n, uint8_t *out, hipStream_t stream) {
    const size_t n_blocks = n / 32;
    if (n_blocks == 0) return hipSuccess;
    const size_t threads = n_blocks * 8;
    const unsigned blocks = (unsigned)((threads + 255) / 256);
    hipLaunchKernelGGL(quantize_q8_0_kernel, dim3(blocks), dim3(256), 0, stream, x, out, n_blocks);
    return hipGetLastError();
}

// ---- dequantize ---------------------------------------------------------

__device__ __forceinline__ float dq_q4_0(const uint8_t *b, uint32_t i) {
    const float d = h2f(ld2(b));
    const uint32_t byte = b[2 + (i >> 1)];
    const int q = (int)((i & 1) ? (byte >> 4) : (byte & 0x0F)) - 8;
    return (float)q * d;  // reference/q4_0.rs:44-45
}

__device__ __forceinline__ float dq_q8_0(const uint8_t *b, uint32_t i) {
    return (float)(int8_t)b[2 + i] * h2f(ld2(b));  // reference/q8_0.rs:40
}

__device__ __forceinline__ float dq_q4_k(const uint8_t *b, uint32_t i) {
    const float d = h2f(ld2(b)), dmin = h2f(ld2(b + 2));
    const uint8_t *s = b + 4;
    const uint32_t j = i >> 5, l = i & 31, g = j >> 1;
    uint32_t sc, mn;  // reference/q4_k.rs:27-49
    if (j < 4) {
        sc = s[j] & 0x3F;
        mn = s[j + 4] & 0x3F;
    } else {
        sc = (s[j + 4] & 0x0F) | ((s[j - 4] >> 6) << 4);
        mn = (s[j + 4] >> 4) | ((s[j] >> 6) << 4);
    }
    const uint32_t byte = b[16 + 32 * g + l];
    const float q = (float)((j & 1) ? (byte >> 4) : (byte & 0x0F));
    const float d1 = d * (float)sc, m1 = dmin * (float)mn;  // reference/q4_k.rs:79-80
    return d1 * q - m1;                                     // reference/q4_k.rs:87
}

__device__ __forceinline__ float dq_q6_k(const uint8_t *b, uint32_t i) {
    const uint32_t hh = i >> 7, r = i & 127, j = r >> 5, l = r & 31, is = l >> 4;
    const uint32_t lb = b[64 * hh + l + 32 * (j & 1)];
    const uint32_t nib = (j >= 2) ? (lb >> 4) : (lb & 0x0F);
    const uint32_t hb = (b[128 + 32 * hh + l] >> (2 * j)) & 3;
    const int q = (int)(nib | (hb << 4)) - 32;  // reference/q6_k.rs:55-60
    const float s = (float)(int8_t)b[192 + 8 * hh + is + 2 * j];
    const float d = h2f(ld2(b + 208));
    return d * s * (float)q;  // reference/q6_k.rs:67-70
}

__device__ __forceinline__ float dq_iq4_xs(const uint8_t *b, uint32_t i) {
    const int8_t kv[16] = {-127, -104, -83, -65, -49, -35, -22, -10, 1, 13, 25, 38, 53, 69, 89, 113};
    const uint32_t sub = i >> 5, k = i & 31;
    const uint32_t scales_h = ld2(b + 2);
    const uint32_t ls_low = (b[4 + (sub >> 1)] >> (4 * (sub & 1))) & 0x0F;
    const uint32_t ls_high = (scales_h >> (2 * sub)) & 3;
    const int ls = (int)(ls_low | (ls_high << 4)) - 32;  // reference/iq4_xs.rs:47-53
    const float scale = h2f(ld2(b)) * (float)ls;         // reference/iq4_xs.rs:81
    const uint32_t byte = b[8 + 16 * sub + (k >> 1)];
    const uint32_t idx = (k & 1) ? (byte >> 4) : (byte & 0x0F);
    return scale * (float)kv[idx];  // reference/iq4_xs.rs:91-92
}

// ---- the formats beyond the first five: element decoders in the reference's operation order ----

__device__ __forceinline__ float dq_q4_1(const uint8_t *b, uint32_t i) {
    const uint32_t byte = b[4 + (i >> 1)];
    const float q = (float)((i & 1) ? (byte >> 4) : (byte & 0x0F));
    return h2f(ld2(b)) * q + h2f(ld2(b + 2));  // reference/q4_1.rs:44-45
}

// q5 of Q5_0 / Q5_1: nibbles at qs, fifth bits in the u32 at qh (reference/q5_0.rs:43-51)
__device__ __forceinline__ uint32_t q5_of(const uint8_t *qh, const uint8_t *qs, uint32_t i) {
    const uint32_t bits = ld4(qh), byte = qs[i & 15];
    const uint32_t nib = i < 16 ? (byte & 0x0F) : (byte >> 4);
    return nib | (((bits >> i) & 1) << 4);
}

__device__ __forceinline__ float dq_q5_0(const uint8_t *b, uint32_t i) {
    return h2f(ld2(b)) * (float)((int)q5_of(b + 2, b + 6, i) - 16);  // reference/q5_0.rs:50-54
}

__device__ __forceinline__ float dq_q5_1(const uint8_t *b, uint32_t i) {
    return h2f(ld2(b)) * (float)q5_of(b + 4, b + 8, i) + h2f(ld2(b + 2));  // reference/q5_1.rs:51-55
}

__device__ __forceinline__ float dq_q8_1(const uint8_t *b, uint32_t i) {
    return h2f(ld2(b)) * (float)(int8_t)b[4 + i];  // reference/q8_1.rs:40-42
}

__device__ __forceinline__ float dq_iq4_nl(const uint8_t *b, uint32_t i) {
    const int8_t kv[16] = {-127, -104, -83, -65, -49, -35, -22, -10, 1, 13, 25, 38, 53, 69, 89, 113};
    const uint32_t byte = b[2 + (i >> 1)];
    return h2f(ld2(b)) * (float)kv[(i & 1) ? (byte >> 4) : (byte & 0x0F)];  // reference/iq4_nl.rs:45-50
}

// column i of a Q2_K / Q3_K super-block: group n, shift 2j, half hf, lane l
__device__ __forceinline__ float dq_q2_k(const uint8_t *b, uint32_t i) {
    const uint32_t is = i >> 4, n = i >> 7, j = (i >> 5) & 3, l = i & 31;
    const uint32_t q = (b[16 + 32 * n + l] >> (2 * j)) & 3;
    const float dl = h2f(ld2(b + 80)) * (float)(b[is] & 0x0F);  // reference/q2_k.rs:56-57
    const float ml = h2f(ld2(b + 82)) * (float)(b[is] >> 4);
    return dl * (float)q - ml;  // reference/q2_k.rs:62
}

__device__ __forceinline__ float dq_q3_k(const uint8_t *b, uint32_t i) {
    const uint32_t is = i >> 4, n = i >> 7, j = (i >> 5) & 3, l = i & 31;
    const uint8_t *s = b + 96;
    uint32_t sc;  // decode_scales, reference/q3_k.rs:30-59
    if (is < 8) {
        sc = s[is] & 0x3F;
    } else if (is < 12) {
        sc = (s[is] & 0x0F) | ((uint32_t)(s[is - 8] >> 6) << 4);
    } else {
        sc = (s[is - 4] >> 4) | ((uint32_t)(s[is - 8] >> 6) << 4);
    }
    const int q_lo = (int)((b[32 + 32 * n + l] >> (2 * j)) & 3);
    const int sub = (b[l] >> (4 * n + j)) & 1 ? 0 : 4;  // reference/q3_k.rs:108-111
    const float dl = h2f(ld2(b + 108)) * (float)((int)sc - 32);
    return dl * (float)(q_lo - sub);
}

__device__ __forceinline__ float dq_q5_k(const uint8_t *b, uint32_t i) {
    const float d = h2f(ld2(b)), dmin = h2f(ld2(b + 2));
    const uint8_t *s = b + 4;
    const uint32_t j = i >> 5, l = i & 31, g = j >> 1;
    uint32_t sc, mn;  // reference/q5_k.rs:27-49
    if (j < 4) {
        sc = s[j] & 0x3F;
        mn = s[j + 4] & 0x3F;
    } else {
        sc = (s[j + 4] & 0x0F) | ((uint32_t)(s[j - 4] >> 6) << 4);
        mn = (s[j + 4] >> 4) | ((uint32_t)(s[j] >> 6) << 4);
    }
    const uint32_t byte = b[48 + 32 * g + l];
    const uint32_t nib = (j & 1) ? (byte >> 4) : (byte & 0x0F);
    const uint32_t q = nib | (((b[16 + l] >> (g + 4 * (j & 1))) & 1) << 4);  // reference/q5_k.rs:84-95
    return d * (float)sc * (float)q - dmin * (float)mn;
}

__global__ __launch_bounds__(256) void dequant_kernel(uint32_t type, const uint8_t *__restrict__ blocks,
                                                     float *__restrict__ out, size_t n_elems,
                                                     uint32_t block_cols, uint32_t block_bytes) {
    const size_t e = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (e >= n_elems) return;
    const uint8_t *b = blocks + (e / block_cols) * block_bytes;
    const uint32_t i = (uint32_t)(e % block_cols);
    float v;
    switch (type) {
    case OXQ_TYPE_Q4_0: v = dq_q4_0(b, i); break;
    case OXQ_TYPE_Q8_0: v = dq_q8_0(b, i); break;
    case OXQ_TYPE_Q4_K: v = dq_q4_k(b, i); break;
    case OXQ_TYPE_Q6_K: v = dq_q6_k(b, i); break;
    case OXQ_TYPE_IQ4_XS: v = dq_iq4_xs(b, i); break;
    case OXQ_TYPE_Q4_1: v = dq_q4_1(b, i); break;
    case OXQ_TYPE_Q5_0: v = dq_q5_0(b, i); break;
    case OXQ_TYPE_Q5_1: v = dq_q5_1(b, i); break;
    case OXQ_TYPE_Q8_1: v = dq_q8_1(b, i); break;
    case OXQ_TYPE_IQ4_NL: v = dq_iq4_nl(b, i); break;
    case OXQ_TYPE_Q2_K: v = dq_q2_k(b, i); break;
    case OXQ_TYPE_Q3_K: v = dq_q3_k(b, i); break;
    default: v = dq_q5_k(b, i); break;
    }
    out[e] = v;
}

hipError_t launch_dequant(uint32_t type, const uint8_t *blocks, size_t n_blocks, float *out, hipStream_t stream) {
    const uint32_t cols = (uint32_t)oxq_block_size(type), bytes = (uint32_t)oxq_block_bytes(type);
    const size_t n = n_blocks * cols;
    if (n == 0) return hipSuccess;
    hipLaunchKernelGGL(dequant_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, stream, type, blocks, out, n,
                       cols, bytes);
    return hipGetLastError();
}

}  // namespace oxq
