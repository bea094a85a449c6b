// Device-side helpers shared by the gfx950 kernels: unaligned vector loads of raw
// GGUF bytes, half -> float, DPP lane exchange and the wave64 sum.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace oxq {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

// GGUF blocks are 18/34/136/144/210 bytes: fields sit at 2-byte (or worse)
// alignment.  gfx950 runs global memory in unaligned-access mode, so a packed
// wrapper yields one global_load_dwordx{2,4} whatever the address.
struct __attribute__((packed, aligned(1))) PackedU4 { u32x4 v; };
struct __attribute__((packed, aligned(1))) PackedU2 { u32x2 v; };
struct __attribute__((packed, aligned(1))) PackedU1 { uint32_t v; };
struct __attribute__((packed, aligned(1))) PackedH1 { uint16_t v; };

__device__ __forceinline__ u32x4 ld16(const uint8_t *p) { return reinterpret_cast<const PackedU4 *>(p)->v; }
__device__ __forceinline__ u32x2 ld8(const uint8_t *p) { return reinterpret_cast<const PackedU2 *>(p)->v; }
__device__ __forceinline__ uint32_t ld4(const uint8_t *p) { return reinterpret_cast<const PackedU1 *>(p)->v; }
__device__ __forceinline__ uint32_t ld2(const uint8_t *p) { return reinterpret_cast<const PackedH1 *>(p)->v; }

// 16 bytes at an address that is only 2-byte aligned, without a sub-dword-misaligned
// vector load (those cost ~15% of streaming bandwidth on gfx950): read five dwords from
// the 4-byte-aligned address at or just below p and funnel-shift by 0, 8, 16 or 24 bits.  The
// fifth dword is only fetched when p is misaligned (otherwise the fourth is re-read), so
// nothing past the dword that holds byte p+15 is touched.
__device__ __forceinline__ u32x4 ld16_h(const uint8_t *p) {
    const uintptr_t a = reinterpret_cast<uintptr_t>(p);
    const uint32_t sh = (uint32_t)(a & 3) * 8;
    const uint32_t *q = reinterpret_cast<const uint32_t *>(a & ~(uintptr_t)3);
    const u32x4 lo = reinterpret_cast<const PackedU4 *>(q)->v;
    const uint32_t hi = q[sh ? 4 : 3];
    u32x4 r;
    r[0] = __builtin_amdgcn_alignbit(lo[1], lo[0], sh);
    r[1] = __builtin_amdgcn_alignbit(lo[2], lo[1], sh);
    r[2] = __builtin_amdgcn_alignbit(lo[3], lo[2], sh);
    r[3] = __builtin_amdgcn_alignbit(hi, lo[3], sh);
    return r;
}

__device__ __forceinline__ void st2(uint8_t *p, uint32_t v) { reinterpret_cast<PackedH1 *>(p)->v = (uint16_t)v; }

// IEEE binary16 bits -> float (v_cvt_f32_f16; subnormals are kept).
__device__ __forceinline__ float h2f(uint32_t bits) {
    return (float)__builtin_bit_cast(_Float16, (uint16_t)bits);
}
// float -> binary16 bits, round to nearest even (v_cvt_f16_f32).
__device__ __forceinline__ uint32_t f2h(float f) {
    return (uint32_t)__builtin_bit_cast(uint16_t, (_Float16)f);
}

// expf as the C library computes it (the routine behind Rust's f32::exp on Linux, which the reference's
// swiglu.rs:18 and moe.rs softmax call): exp(x) = 2^(k/32) * 2^(r/32) in double with a 32-entry table of 2^(i/32) and a
// cubic in r, one rounding to float at the end.  The device's own expf differs from it in the last place for a
// large share of arguments, and a last-place difference of h can move a Q8_0 byte of the down projection's input
// by a whole step; this form agrees with the host's on all but a few arguments in 10^8.
static __device__ __constant__ const uint64_t EXP2_TAB[32] = {
    0x3ff0000000000000ull, 0x3fefd9b0d3158574ull, 0x3fefb5586cf9890full, 0x3fef9301d0125b51ull, 0x3fef72b83c7d517bull,
    0x3fef54873168b9aaull, 0x3fef387a6e756238ull, 0x3fef1e9df51fdee1ull, 0x3fef06fe0a31b715ull, 0x3feef1a7373aa9cbull,
    0x3feedea64c123422ull, 0x3feece086061892dull, 0x3feebfdad5362a27ull, 0x3feeb42b569d4f82ull, 0x3feeab07dd485429ull,
    0x3feea47eb03a5585ull, 0x3feea09e667f3bcdull, 0x3fee9f75e8ec5f74ull, 0x3feea11473eb0187ull, 0x3feea589994cce13ull,
    0x3feeace5422aa0dbull, 0x3feeb737b0cdc5e5ull, 0x3feec49182a3f090ull, 0x3feed503b23e255dull, 0x3feee89f995ad3adull,
    0x3feeff76f2fb5e47ull, 0x3fef199bdd85529cull, 0x3fef3720dcef9069ull, 0x3fef5818dcfba487ull, 0x3fef7c97337b9b5full,
    0x3fefa4afa2a490daull, 0x3fefd0765b6e4540ull};  // bits of 2^(i/32) minus i << 47
__device__ __forceinline__ float expf_libm(float x) {
    if (x > 0x1.62e42ep6f) return __builtin_inff();  // overflow
    if (x < -0x1.9fe368p6f) return 0.0f;             // below the smallest subnormal
    constexpr double N = 32.0, INV_LN2_N = 0x1.71547652b82fep+0 * N, SHIFT = 0x1.8p52;
    constexpr double C0 = 0x1.c6af84b912394p-5 / N / N / N, C1 = 0x1.ebfce50fac4f3p-3 / N / N, C2 = 0x1.62e42ff0c52d6p-1 / N;
    double z = INV_LN2_N * (double)x, kd = z + SHIFT;  // kd: z rounded to an integer, in the low mantissa bits
    const uint64_t ki = __builtin_bit_cast(uint64_t, kd);
    kd -= SHIFT;
    const double r = z - kd;
    const double s = __builtin_bit_cast(double, EXP2_TAB[ki & 31] + (ki << 47));
    z = C0 * r + C1;
    double y = C2 * r + 1.0;
    y = z * (r * r) + y;
    return (float)(y * s);
}

__device__ __forceinline__ int sdot4(uint32_t a, uint32_t b, int c) {
    return __builtin_amdgcn_sdot4((int)a, (int)b, c, false);
}

// DPP controls: quad_perm [1,0,3,2] = 0xB1, [2,3,0,1] = 0x4E, row_ror:n = 0x120+n.
template <int CTRL> __device__ __forceinline__ int dpp_i(int v) {
    return __builtin_amdgcn_update_dpp(0, v, CTRL, 0xF, 0xF, true);
}
template <int CTRL> __device__ __forceinline__ float dpp_f(float v) {
    return __builtin_bit_cast(float, dpp_i<CTRL>(__builtin_bit_cast(int, v)));
}
// Value held by lane ^ 1 / lane ^ 2.
__device__ __forceinline__ int xor1_i(int v) { return dpp_i<0xB1>(v); }
__device__ __forceinline__ int xor2_i(int v) { return dpp_i<0x4E>(v); }

__device__ __forceinline__ float readlane_f(float v, int lane) {
    return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), lane));
}

// Sum over the 64 lanes, same value and same order in every lane: butterflies in
// each quad, rotations inside each row of 16, then the four row sums.
__device__ __forceinline__ float wave_sum(float v) {
    v += dpp_f<0xB1>(v);
    v += dpp_f<0x4E>(v);
    v += dpp_f<0x124>(v);
    v += dpp_f<0x128>(v);
    float r0 = readlane_f(v, 0), r1 = readlane_f(v, 16), r2 = readlane_f(v, 32), r3 = readlane_f(v, 48);
    return (r0 + r1) + (r2 + r3);
}

__device__ __forceinline__ uint64_t max_u64(uint64_t a, uint64_t b) { return a > b ? a : b; }
// Maximum over the 64 lanes of a wave, the same value in every lane; no LDS, no barrier.
__device__ __forceinline__ uint32_t wave_max_u32(uint32_t v) {
    v = max(v, (uint32_t)dpp_i<0xB1>((int)v));   // quad_perm [1,0,3,2]
    v = max(v, (uint32_t)dpp_i<0x4E>((int)v));   // quad_perm [2,3,0,1]
    v = max(v, (uint32_t)dpp_i<0x124>((int)v));  // row_ror:4
    v = max(v, (uint32_t)dpp_i<0x128>((int)v));  // row_ror:8
    const uint32_t r0 = (uint32_t)__builtin_amdgcn_readlane((int)v, 0), r1 = (uint32_t)__builtin_amdgcn_readlane((int)v, 16);
    const uint32_t r2 = (uint32_t)__builtin_amdgcn_readlane((int)v, 32), r3 = (uint32_t)__builtin_amdgcn_readlane((int)v, 48);
    return max(max(r0, r1), max(r2, r3));
}
// The same for 64-bit keys, as two 32-bit maxima: the largest upper half, then the largest lower half among
// the lanes that hold it (fewer instructions than carrying 64-bit compares through the DPP steps).
__device__ __forceinline__ uint64_t wave_max_u64(uint64_t v) {
    const uint32_t hi = (uint32_t)(v >> 32), lo = (uint32_t)v;
    const uint32_t mh = wave_max_u32(hi);
    const uint32_t ml = wave_max_u32(hi == mh ? lo : 0u);
    return ((uint64_t)mh << 32) | ml;
}

// Top-k keys: the order-preserving bits of a float, then the complement of its index -- one unsigned maximum decides
// value and tie (the lower index first) at once; NaN ranks below everything.
__device__ __forceinline__ uint64_t topk_key(float v, uint32_t index) {
    uint32_t b = __builtin_bit_cast(uint32_t, v);
    b = (b & 0x80000000u) ? ~b : (b | 0x80000000u);  // unsigned order == float order
    if (v != v) b = 0;                                // NaN ranks below everything
    return ((uint64_t)b << 32) | (uint64_t)(0xFFFFFFFFu - index);
}
__device__ __forceinline__ float topk_value(uint64_t key) {
    uint32_t b = (uint32_t)(key >> 32);
    b = (b & 0x80000000u) ? (b & 0x7FFFFFFFu) : ~b;
    return __builtin_bit_cast(float, b);
}

}  // namespace oxq
