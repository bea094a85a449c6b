// The Q8_0 block encoder as a device function, shared by the plain quantizer and by the kernels
// that produce their activations themselves (SwiGLU, RMSNorm) and quantize them on the way out.
// Bit-exact twin of encode_q8_0_block in the reference
// (crates/oxillama-quant/src/quantize.rs:190-210).
#pragma once
#include "oxq_device.hpp"

namespace oxq {

// Four consecutive floats at a 16-byte aligned address.
__device__ __forceinline__ void load4(float (&v)[4], const float *p) {
    const u32x4 raw = ld16(reinterpret_cast<const uint8_t *>(p));
    for (int i = 0; i < 4; i++) {
        const uint32_t bits = raw[i];  // copy out first: bit_cast must not see the vector element lvalue
        v[i] = __builtin_bit_cast(float, bits);
    }
}

// Eight consecutive lanes (j = 0..7, aligned to a multiple of 8 in the wave) hold one block of
// 32 floats, four each; all 64 lanes of the wave must call this together.  Writes the 34-byte
// block at ob when valid.
__device__ __forceinline__ void encode_q8_0_lanes(const float (&v)[4], bool valid, uint8_t *ob, uint32_t j) {
    float m = 0.0f;
    for (int i = 0; i < 4; i++) m = fmaxf(m, fabsf(v[i]));
    m = fmaxf(m, dpp_f<0xB1>(m));
    m = fmaxf(m, dpp_f<0x4E>(m));
    m = fmaxf(m, __shfl_xor(m, 4, 64));  // max is exact: any order gives the fold of quantize.rs:194
    const float d = m / 127.0f;                        // quantize.rs:197
    const float id = (d != 0.0f) ? 1.0f / d : 0.0f;    // quantize.rs:198
    uint32_t packed = 0;
    for (int i = 0; i < 4; i++) {
        int q = (int)roundf(v[i] * id);  // quantize.rs:206 (round half away from zero)
        q = q < -128 ? -128 : (q > 127 ? 127 : q);
        packed |= ((uint32_t)q & 0xFFu) << (8 * i);
    }
    if (valid) {
        if (j == 0) st2(ob, f2h(d));  // quantize.rs:201
        reinterpret_cast<PackedU1 *>(ob + 2 + 4 * j)->v = packed;
    }
}

}  // namespace oxq
