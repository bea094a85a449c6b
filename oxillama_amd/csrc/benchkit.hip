// Measurement helpers (not part of the quantized-matmul ABI): a plain copy kernel of
// known size, used to scale rocprofv3's FETCH_SIZE / WRITE_SIZE counters, a
// streaming read kernel that marks the practical HBM read ceiling for a given
// footprint and launch shape, and a kernel of nothing but int8 MFMAs on register
// operands, which marks what the matrix cores deliver when nothing else is in the way.
#include <hip/hip_runtime.h>
#include <stdint.h>

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

__global__ __launch_bounds__(256) void benchkit_copy_kernel(const u32x4 *__restrict__ src, u32x4 *__restrict__ dst,
                                                           size_t n16) {
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n16; i += stride) dst[i] = src[i];
}

// Each thread reads `unroll` independent 16-byte chunks per trip and xors them; one
// dword per wave is written so the loads cannot be dropped.
template <int UNROLL>
__global__ __launch_bounds__(256) void benchkit_read_kernel(const u32x4 *__restrict__ src, uint32_t *__restrict__ out,
                                                           size_t n16) {
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    u32x4 acc = {0, 0, 0, 0};
    for (; i + (UNROLL - 1) * stride < n16; i += UNROLL * stride) {
        u32x4 v[UNROLL];
#pragma unroll
        for (int u = 0; u < UNROLL; u++) v[u] = src[i + u * stride];
#pragma unroll
        for (int u = 0; u < UNROLL; u++) acc ^= v[u];
    }
    for (; i < n16; i += stride) acc ^= src[i];
    uint32_t r = acc.x ^ acc.y ^ acc.z ^ acc.w;
    if (r == 0x9E3779B9u) out[blockIdx.x] = r;  // practically never: keeps the loads alive
}

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));

// Four independent accumulator chains of v_mfma_i32_32x32x32_i8 per wave, `iters` rounds.
__global__ __launch_bounds__(256) void benchkit_mfma_i8_kernel(int *__restrict__ out, int iters) {
    const int lane = threadIdx.x;
    v4i a = {lane, lane * 3, lane * 5, lane * 7}, b = {lane ^ 21, lane * 11, lane * 13, lane * 17};
    v16i acc[4];
    for (int c = 0; c < 4; c++)
        for (int i = 0; i < 16; i++) acc[c][i] = 0;
    for (int it = 0; it < iters; it++) {
#pragma unroll
        for (int c = 0; c < 4; c++) acc[c] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a, b, acc[c], 0, 0, 0);
    }
    int r = 0;
    for (int c = 0; c < 4; c++)
        for (int i = 0; i < 16; i++) r ^= acc[c][i];
    out[(size_t)blockIdx.x * blockDim.x + threadIdx.x] = r;
}

extern "C" {

// blocks x 4 waves x iters x 4 MFMAs of 2 * 32 * 32 * 32 int8 operations; out: blocks * 256 ints.
int oxq_benchkit_mfma_i8(void *out, unsigned blocks, int iters, void *stream) {
    hipLaunchKernelGGL(benchkit_mfma_i8_kernel, dim3(blocks), dim3(256), 0, (hipStream_t)stream, (int *)out, iters);
    return (int)hipGetLastError();
}

int oxq_benchkit_copy(const void *src, void *dst, size_t bytes, unsigned blocks, void *stream) {
    hipLaunchKernelGGL(benchkit_copy_kernel, dim3(blocks), dim3(256), 0, (hipStream_t)stream, (const u32x4 *)src,
                       (u32x4 *)dst, bytes / 16);
    return (int)hipGetLastError();
}

int oxq_benchkit_read(const void *src, void *out, size_t bytes, unsigned blocks, int unroll, void *stream) {
    const u32x4 *s = (const u32x4 *)src;
    uint32_t *o = (uint32_t *)out;
    hipStream_t st = (hipStream_t)stream;
    switch (unroll) {
    case 1: hipLaunchKernelGGL(benchkit_read_kernel<1>, dim3(blocks), dim3(256), 0, st, s, o, bytes / 16); break;
    case 2: hipLaunchKernelGGL(benchkit_read_kernel<2>, dim3(blocks), dim3(256), 0, st, s, o, bytes / 16); break;
    case 4: hipLaunchKernelGGL(benchkit_read_kernel<4>, dim3(blocks), dim3(256), 0, st, s, o, bytes / 16); break;
    default: hipLaunchKernelGGL(benchkit_read_kernel<8>, dim3(blocks), dim3(256), 0, st, s, o, bytes / 16); break;
    }
    return (int)hipGetLastError();
}
}
