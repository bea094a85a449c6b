// Measurement helpers (not part of the quantized-matmul ABI): a plain copy kernel of
// known size, used to scale rocprofv3's FETCH_SIZE / WRITE_SIZE counters, and a
// streaming read kernel that marks the practical HBM read ceiling for a given
// footprint and launch shape.
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

extern "C" {

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
