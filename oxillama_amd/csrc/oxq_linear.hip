// The callers' glue around the quantized matvec, on the device (gfx950): what
// QuantLinear::forward and the dense feed-forward block of the reference do between two
// projections, fused with the Q8_0 quantizer of the next projection's input so that fp32
// activations make one trip through memory.
//
//   swiglu_quantize_kernel   swiglu_inplace (crates/oxillama-arch/src/common/swiglu.rs:15-21)
//                            + quantize_f32_to_q8_0 (crates/oxillama-quant/src/quantize.rs:58)
//   rmsnorm_quantize_kernel  RmsNorm::forward_to (crates/oxillama-arch/src/common/rms_norm.rs:49-66)
//                            + quantize_f32_to_q8_0
//   lora_down / lora_up      LoraAdapter::apply (crates/oxillama-quant/src/lora.rs:83-124)
//
// All of it is HBM/latency-bound elementwise work on vectors of a few thousand floats.
#include "oxq_device.hpp"
#include "oxq_internal.hpp"
#include "oxq_q8_encode.hpp"

namespace oxq {

// h = silu(gate) * up, in the reference's operation order: sigmoid = 1 / (1 + exp(-g));
// h = (g * sigmoid) * u.  Eight lanes per 32-float block, as in the quantizer.
__global__ __launch_bounds__(256) void swiglu_quantize_kernel(const float *__restrict__ gate,
                                                             const float *__restrict__ up, float *__restrict__ h_out,
                                                             uint8_t *__restrict__ out, size_t n_blocks) {
    const size_t t = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const size_t blk = t >> 3;
    const uint32_t j = (uint32_t)(t & 7);
    const bool valid = blk < n_blocks;
    float v[4] = {0.0f, 0.0f, 0.0f, 0.0f};
    if (valid) {
        float g[4], u[4];
        load4(g, gate + blk * 32 + 4 * j);
        load4(u, up + blk * 32 + 4 * j);
        for (int i = 0; i < 4; i++) {
            const float sigmoid = 1.0f / (1.0f + expf_libm(-g[i]));  // swiglu.rs:18
            v[i] = g[i] * sigmoid * u[i];                       // swiglu.rs:19
        }
        if (h_out) {
            float *hp = h_out + blk * 32 + 4 * j;
            for (int i = 0; i < 4; i++) hp[i] = v[i];
        }
    }
    if (out) encode_q8_0_lanes(v, valid, out + blk * 34, j);
}

hipError_t launch_swiglu_quantize(const float *gate, const float *up, size_t n, float *h, uint8_t *out,
                                  hipStream_t stream) {
    const size_t n_blocks = n / 32;
    if (n_blocks == 0) return hipSuccess;
    const unsigned blocks = (unsigned)((n_blocks * 8 + 255) / 256);
    hipLaunchKernelGGL(swiglu_quantize_kernel, dim3(blocks), dim3(256), 0, stream, gate, up, h, out, n_blocks);
    return hipGetLastError();
}

// One work group per row of n floats (n % 32 == 0).  rms = sqrt(sum(x^2)/n + eps); y = (x *
// (1/rms)) * weight.  The sum of squares is formed per lane, per wave, then over the four waves
// (the reference adds sequentially; fp32 results agree to rounding).  The row is read twice (the
// second pass hits L2), so any n fits.
__global__ __launch_bounds__(256) void rmsnorm_quantize_kernel(const float *__restrict__ x,
                                                              const float *__restrict__ weight, float eps, uint32_t n,
                                                              float *__restrict__ y_out, uint8_t *__restrict__ out) {
    __shared__ float wave_part[4];
    const size_t row = blockIdx.x;
    const float *xr = x + row * n;
    const uint32_t n_chunks = n / 4;  // 16-byte pieces
    float ss = 0.0f;
    for (uint32_t c = threadIdx.x; c < n_chunks; c += 256) {
        float v[4];
        load4(v, xr + 4 * c);
        for (int i = 0; i < 4; i++) ss += v[i] * v[i];  // rms_norm.rs:56-58
    }
    ss = wave_sum(ss);
    if ((threadIdx.x & 63) == 0) wave_part[threadIdx.x >> 6] = ss;
    __syncthreads();
    const float sum_sq = (wave_part[0] + wave_part[1]) + (wave_part[2] + wave_part[3]);
    const float rms = sqrtf(sum_sq / (float)n + eps);  // rms_norm.rs:59
    const float inv_rms = 1.0f / rms;                  // rms_norm.rs:60
    // every wave walks whole trips so that the eight lanes of a block stay together
    const uint32_t trips = (n_chunks + 255) / 256;
    for (uint32_t tr = 0; tr < trips; tr++) {
        const uint32_t c = tr * 256 + threadIdx.x;
        const bool valid = c < n_chunks;
        float v[4] = {0.0f, 0.0f, 0.0f, 0.0f};
        if (valid) {
            float xv[4], wv[4];
            load4(xv, xr + 4 * c);
            load4(wv, weight + 4 * c);
            for (int i = 0; i < 4; i++) v[i] = xv[i] * inv_rms * wv[i];  // rms_norm.rs:63
            if (y_out) {
                float *yp = y_out + row * n + 4 * c;
                for (int i = 0; i < 4; i++) yp[i] = v[i];
            }
        }
        if (out) encode_q8_0_lanes(v, valid, out + (row * (n / 32) + (c >> 3)) * 34, c & 7);
    }
}

hipError_t launch_rmsnorm_quantize(const float *x, const float *weight, float eps, size_t rows, uint32_t n, float *y,
                                   uint8_t *out, hipStream_t stream) {
    if (rows == 0 || n == 0) return hipSuccess;
    hipLaunchKernelGGL(rmsnorm_quantize_kernel, dim3((unsigned)rows), dim3(256), 0, stream, x, weight, eps, n, y, out);
    return hipGetLastError();
}

// r[i] = sum_j a[i][j] * x[j]: one work group per rank row (lora.rs:97-107).
__global__ __launch_bounds__(256) void lora_down_kernel(const float *__restrict__ a, const float *__restrict__ x,
                                                       float *__restrict__ r, uint32_t in_features) {
    __shared__ float wave_part[4];
    const float *ar = a + (size_t)blockIdx.x * in_features;
    float acc = 0.0f;
    for (uint32_t j = threadIdx.x; j < in_features; j += 256) acc += ar[j] * x[j];
    acc = wave_sum(acc);
    if ((threadIdx.x & 63) == 0) wave_part[threadIdx.x >> 6] = acc;
    __syncthreads();
    if (threadIdx.x == 0) r[blockIdx.x] = (wave_part[0] + wave_part[1]) + (wave_part[2] + wave_part[3]);
}

// out[i] += (sum_j b[i][j] * r[j]) * scale, j in ascending order from 0.0 as the reference's
// iterator sum does (lora.rs:109-121).
__global__ __launch_bounds__(256) void lora_up_kernel(const float *__restrict__ b, const float *__restrict__ r,
                                                     float *__restrict__ out, uint32_t out_features, uint32_t rank,
                                                     float scale) {
    const uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= out_features) return;
    const float *br = b + (size_t)i * rank;
    float s = 0.0f;
    for (uint32_t j = 0; j < rank; j++) s += br[j] * r[j];
    out[i] += s * scale;
}

hipError_t launch_lora_apply(const float *a, const float *b, float *r, uint32_t rank, float scale, const float *x,
                             float *out, uint32_t out_features, uint32_t in_features, hipStream_t stream) {
    if (rank == 0 || out_features == 0) return hipSuccess;
    hipLaunchKernelGGL(lora_down_kernel, dim3(rank), dim3(256), 0, stream, a, x, r, in_features);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return e;
    hipLaunchKernelGGL(lora_up_kernel, dim3((out_features + 255) / 256), dim3(256), 0, stream, b, r, out, out_features,
                       rank, scale);
    return hipGetLastError();
}

}  // namespace oxq
