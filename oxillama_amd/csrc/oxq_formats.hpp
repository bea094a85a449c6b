// Per-format lane work for the Q8_0-activation GEMV on gfx950.
//
// A row of n_cols weights is cut into "units"; lane l of a wave owns unit
// 64*step + l.  For each format this file says which raw GGUF bytes the lane
// loads for its unit (Wt), which Q8_0 activation bytes it keeps in registers for
// every row (Act), and how the exact int32 group sums and the fp32 term are
// formed from them.  Byte layouts follow the reference decoders cited below
// (Q/ = crates/oxillama-quant/src in the reference tree).
//
// Integer groups (the unit of the bit-exact check): 32 weights = one Q8_0
// activation block for Q4_0 / Q8_0 / Q4_K / IQ4_XS, 16 weights for Q6_K.
#pragma once
#include "oxq_device.hpp"

namespace oxq {

constexpr uint32_t Q8_BLOCK_BYTES = 34;  // Q/traits.rs:12: f16 d + 32 x i8

// ---------------------------------------------------------------------------
// Q4_K, Q/reference/q4_k.rs:27-99,218-333.  144 B = d, dmin (f16), 12 B packed
// 6-bit scales/mins, 128 B nibbles.  Unit = one 16-byte chunk c (0..7) of qs:
// low nibbles are 16 weights of sub-block 2g, high nibbles 16 weights of
// sub-block 2g+1 (g = c/2), at bytes 16h.. of those activation blocks (h = c&1).
// The two lanes of a pair (h = 0, 1) add their halves; lane h then owns the fp32
// term of sub-block 2g+h = c.
struct FmtQ4K {
    static constexpr uint32_t BLOCK_BYTES = 144, BLOCK_COLS = 256, UNIT_COLS = 32;
    struct Lane {
        uint32_t c, h, sh;
        bool upper;
    };
    struct Act {
        u32x4 lo, hi;
        float d_a, fasum;
    };
    struct Wt {
        u32x4 hdr, qs;
    };
    static __device__ __forceinline__ Lane lane_consts(uint32_t lane) {
        Lane k;
        k.c = lane & 7;
        k.h = lane & 1;
        k.sh = (k.c & 3) * 8;
        k.upper = k.c >= 4;
        return k;
    }
    static __device__ __forceinline__ void load_act(Act &a, const uint8_t *A, uint32_t u, bool valid,
                                                    const Lane &k) {
        const uint32_t b = u >> 3, g = k.c >> 1;
        const uint8_t *blo = A + (size_t)(8 * b + 2 * g) * Q8_BLOCK_BYTES;
        const uint8_t *bhi = blo + Q8_BLOCK_BYTES;
        const u32x4 z = {0, 0, 0, 0};
        a.lo = valid ? ld16(blo + 2 + 16 * k.h) : z;
        a.hi = valid ? ld16(bhi + 2 + 16 * k.h) : z;
        int slo = 0, shi = 0;
        for (int i = 0; i < 4; i++) {
            slo = sdot4(a.lo[i], 0x01010101u, slo);
            shi = sdot4(a.hi[i], 0x01010101u, shi);
        }
        slo += xor1_i(slo);
        shi += xor1_i(shi);
        a.fasum = (float)(k.h ? shi : slo);
        a.d_a = valid ? h2f(ld2(k.h ? bhi : blo)) : 0.0f;
    }
    static __device__ __forceinline__ void load_w(Wt &w, const uint8_t *row, uint32_t u, bool valid,
                                                  const Lane &k) {
        const uint8_t *blk = row + (size_t)(u >> 3) * BLOCK_BYTES;
        const u32x4 z = {0, 0, 0, 0};
        w.hdr = valid ? ld16(blk) : z;
        w.qs = valid ? ld16(blk + 16 + 16 * k.c) : z;
    }
    template <bool DUMP>
    static __device__ __forceinline__ float dot(const Wt &w, const Act &a, const Lane &k, int32_t *sums,
                                                uint32_t u, bool valid) {
        int plo = 0, phi = 0;
        for (int i = 0; i < 4; i++) {
            plo = sdot4(w.qs[i] & 0x0F0F0F0Fu, a.lo[i], plo);
            phi = sdot4((w.qs[i] >> 4) & 0x0F0F0F0Fu, a.hi[i], phi);
        }
        plo += xor1_i(plo);
        phi += xor1_i(phi);
        const int isum = k.h ? phi : plo;
        // 6-bit scale / min of sub-block j = c (decode_scales_mins, q4_k.rs:27-49)
        const uint32_t s_a = (w.hdr[1] >> k.sh) & 0xFF, s_b = (w.hdr[2] >> k.sh) & 0xFF,
                       s_c = (w.hdr[3] >> k.sh) & 0xFF;
        const uint32_t sc = k.upper ? ((s_c & 0x0F) | ((s_a >> 6) << 4)) : (s_a & 0x3F);
        const uint32_t mn = k.upper ? ((s_c >> 4) | ((s_b >> 6) << 4)) : (s_b & 0x3F);
        const float d = h2f(w.hdr[0] & 0xFFFF), dmin = h2f(w.hdr[0] >> 16);
        const float da = d * (float)sc, m = dmin * (float)mn;  // q4_k.rs:280-281
        if (DUMP && valid) sums[u] = isum;
        return (da * (float)isum - m * a.fasum) * a.d_a;  // q4_k.rs:307 / avx2/q4_k.rs:329
    }
};

// ---------------------------------------------------------------------------
// Q6_K, Q/reference/q6_k.rs:39-72,246-351.  210 B = ql[128], qh[64], i8
// scales[16], f16 d.  Unit = (half hh, sixteen is) of a super-block: bytes
// ql[64hh+16is..+16], ql[64hh+32+16is..+16], qh[32hh+16is..+16] give four
// 16-weight sub-blocks at columns 128hh + 32k + 16is (k = 0..3), scale index
// 8hh + is + 2k, activation block 8b + 4hh + k bytes 16is..+16.
struct FmtQ6K {
    static constexpr uint32_t BLOCK_BYTES = 210, BLOCK_COLS = 256, UNIT_COLS = 64;
    struct Lane {
        uint32_t hh, is;
    };
    struct Act {
        u32x4 q[4];
        float d_a[4];
        int asum32[4];  // 32 * sum of the 16 activation bytes
    };
    struct Wt {
        u32x4 ql0, ql1, qh;
        u32x2 sc;
        uint32_t d;
    };
    static __device__ __forceinline__ Lane lane_consts(uint32_t lane) {
        Lane k;
        k.hh = (lane >> 1) & 1;
        k.is = lane & 1;
        return k;
    }
    static __device__ __forceinline__ void load_act(Act &a, const uint8_t *A, uint32_t u, bool valid,
                                                    const Lane &k) {
        const uint32_t b = u >> 2;
        const u32x4 z = {0, 0, 0, 0};
        for (int j = 0; j < 4; j++) {
            const uint8_t *blk = A + (size_t)(8 * b + 4 * k.hh + j) * Q8_BLOCK_BYTES;
            a.q[j] = valid ? ld16(blk + 2 + 16 * k.is) : z;
            a.d_a[j] = valid ? h2f(ld2(blk)) : 0.0f;
            int s = 0;
            for (int i = 0; i < 4; i++) s = sdot4(a.q[j][i], 0x01010101u, s);
            a.asum32[j] = 32 * s;
        }
    }
    static __device__ __forceinline__ void load_w(Wt &w, const uint8_t *row, uint32_t u, bool valid,
                                                  const Lane &k) {
        const uint8_t *blk = row + (size_t)(u >> 2) * BLOCK_BYTES;
        const u32x4 z = {0, 0, 0, 0};
        const u32x2 z2 = {0, 0};
        w.ql0 = valid ? ld16(blk + 64 * k.hh + 16 * k.is) : z;
        w.ql1 = valid ? ld16(blk + 64 * k.hh + 32 + 16 * k.is) : z;
        w.qh = valid ? ld16(blk + 128 + 32 * k.hh + 16 * k.is) : z;
        w.sc = valid ? ld8(blk + 192 + 8 * k.hh) : z2;
        w.d = valid ? ld2(blk + 208) : 0u;
    }
    template <bool DUMP>
    static __device__ __forceinline__ float dot(const Wt &w, const Act &a, const Lane &k, int32_t *sums,
                                                uint32_t u, bool valid) {
        int p0 = 0, p1 = 0, p2 = 0, p3 = 0;
        for (int i = 0; i < 4; i++) {
            const uint32_t l0 = w.ql0[i], l1 = w.ql1[i], h = w.qh[i];
            // q6_k.rs:55-60, four bytes at a time
            const uint32_t q0 = (l0 & 0x0F0F0F0Fu) | ((h << 4) & 0x30303030u);
            const uint32_t q1 = (l1 & 0x0F0F0F0Fu) | ((h << 2) & 0x30303030u);
            const uint32_t q2 = ((l0 >> 4) & 0x0F0F0F0Fu) | (h & 0x30303030u);
            const uint32_t q3 = ((l1 >> 4) & 0x0F0F0F0Fu) | ((h >> 2) & 0x30303030u);
            p0 = sdot4(q0, a.q[0][i], p0);
            p1 = sdot4(q1, a.q[1][i], p1);
            p2 = sdot4(q2, a.q[2][i], p2);
            p3 = sdot4(q3, a.q[3][i], p3);
        }
        const int isum[4] = {p0 - a.asum32[0], p1 - a.asum32[1], p2 - a.asum32[2], p3 - a.asum32[3]};
        // scales[8hh + is + 2j]: bytes is, is+2 of sc[0], then of sc[1]
        const uint32_t s0 = w.sc[0] >> (8 * k.is), s1 = w.sc[1] >> (8 * k.is);
        const int scv[4] = {(int)(int8_t)(s0 & 0xFF), (int)(int8_t)((s0 >> 16) & 0xFF),
                            (int)(int8_t)(s1 & 0xFF), (int)(int8_t)((s1 >> 16) & 0xFF)};
        const float d = h2f(w.d);
        float t = 0.0f;
        for (int j = 0; j < 4; j++) {
            const float s = d * (float)scv[j];  // q6_k.rs:285
            t += s * (float)isum[j] * a.d_a[j];
            if (DUMP && valid) sums[16 * (u >> 2) + 8 * k.hh + 2 * j + k.is] = isum[j];
        }
        return t;
    }
};

// ---------------------------------------------------------------------------
// Q8_0 weights, Q/reference/q8_0.rs:36-41; fused form Q/simd/avx2/q8_0.rs:205,242.
// Unit = one 34-byte block against the activation block of the same index.
struct FmtQ8_0 {
    static constexpr uint32_t BLOCK_BYTES = 34, BLOCK_COLS = 32, UNIT_COLS = 32;
    struct Lane {};
    struct Act {
        u32x4 q0, q1;
        float d_a;
    };
    struct Wt {
        u32x4 q0, q1;
        uint32_t d;
    };
    static __device__ __forceinline__ Lane lane_consts(uint32_t) { return Lane{}; }
    static __device__ __forceinline__ void load_act(Act &a, const uint8_t *A, uint32_t u, bool valid,
                                                    const Lane &) {
        const uint8_t *blk = A + (size_t)u * Q8_BLOCK_BYTES;
        const u32x4 z = {0, 0, 0, 0};
        a.q0 = valid ? ld16(blk + 2) : z;
        a.q1 = valid ? ld16(blk + 18) : z;
        a.d_a = valid ? h2f(ld2(blk)) : 0.0f;
    }
    static __device__ __forceinline__ void load_w(Wt &w, const uint8_t *row, uint32_t u, bool valid,
                                                  const Lane &) {
        const uint8_t *blk = row + (size_t)u * BLOCK_BYTES;
        const u32x4 z = {0, 0, 0, 0};
        w.q0 = valid ? ld16(blk + 2) : z;
        w.q1 = valid ? ld16(blk + 18) : z;
        w.d = valid ? ld2(blk) : 0u;
    }
    template <bool DUMP>
    static __device__ __forceinline__ float dot(const Wt &w, const Act &a, const Lane &, int32_t *sums,
                                                uint32_t u, bool valid) {
        int p = 0;
        for (int i = 0; i < 4; i++) {
            p = sdot4(w.q0[i], a.q0[i], p);
            p = sdot4(w.q1[i], a.q1[i], p);
        }
        if (DUMP && valid) sums[u] = p;
        const float scale = h2f(w.d) * a.d_a;  // avx2/q8_0.rs:205
        return scale * (float)p;               // avx2/q8_0.rs:242
    }
};

// Nibble-interleaved formats (Q4_0, IQ4_XS): byte i of a 16-byte payload holds
// weight 2i (low nibble) and 2i+1 (high nibble).  Masking a dword gives the four
// even-column and the four odd-column weights of 8 consecutive columns, so the
// activation bytes are split once per lane into even/odd dwords instead.
__device__ __forceinline__ void split_even_odd(const u32x4 &q0, const u32x4 &q1, uint32_t ev[4],
                                               uint32_t od[4]) {
    const uint32_t a[8] = {q0[0], q0[1], q0[2], q0[3], q1[0], q1[1], q1[2], q1[3]};
    for (int i = 0; i < 4; i++) {
        ev[i] = __builtin_amdgcn_perm(a[2 * i + 1], a[2 * i], 0x06040200u);
        od[i] = __builtin_amdgcn_perm(a[2 * i + 1], a[2 * i], 0x07050301u);
    }
}

// ---------------------------------------------------------------------------
// Q4_0, Q/reference/q4_0.rs:37-46; fused form Q/simd/avx2/q4_0.rs:211,265.
// Unit = one 18-byte block.  sum (q-8)*a = sum q*a - 8*sum a.
struct FmtQ4_0 {
    static constexpr uint32_t BLOCK_BYTES = 18, BLOCK_COLS = 32, UNIT_COLS = 32;
    struct Lane {};
    struct Act {
        uint32_t ev[4], od[4];
        float d_a;
        int asum8;
    };
    struct Wt {
        u32x4 q;
        uint32_t d;
    };
    static __device__ __forceinline__ Lane lane_consts(uint32_t) { return Lane{}; }
    static __device__ __forceinline__ void load_act(Act &a, const uint8_t *A, uint32_t u, bool valid,
                                                    const Lane &) {
        const uint8_t *blk = A + (size_t)u * Q8_BLOCK_BYTES;
        const u32x4 z = {0, 0, 0, 0};
        const u32x4 q0 = valid ? ld16(blk + 2) : z, q1 = valid ? ld16(blk + 18) : z;
        split_even_odd(q0, q1, a.ev, a.od);
        int s = 0;
        for (int i = 0; i < 4; i++) {
            s = sdot4(q0[i], 0x01010101u, s);
            s = sdot4(q1[i], 0x01010101u, s);
        }
        a.asum8 = 8 * s;
        a.d_a = valid ? h2f(ld2(blk)) : 0.0f;
    }
    static __device__ __forceinline__ void load_w(Wt &w, const uint8_t *row, uint32_t u, bool valid,
                                                  const Lane &) {
        const uint8_t *blk = row + (size_t)u * BLOCK_BYTES;
        const u32x4 z = {0, 0, 0, 0};
        w.q = valid ? ld16(blk + 2) : z;
        w.d = valid ? ld2(blk) : 0u;
    }
    template <bool DUMP>
    static __device__ __forceinline__ float dot(const Wt &w, const Act &a, const Lane &, int32_t *sums,
                                                uint32_t u, bool valid) {
        int p = 0;
        for (int i = 0; i < 4; i++) {
            p = sdot4(w.q[i] & 0x0F0F0F0Fu, a.ev[i], p);
            p = sdot4((w.q[i] >> 4) & 0x0F0F0F0Fu, a.od[i], p);
        }
        p -= a.asum8;
        if (DUMP && valid) sums[u] = p;
        const float scale = h2f(w.d) * a.d_a;  // avx2/q4_0.rs:211
        return scale * (float)p;               // avx2/q4_0.rs:265
    }
};

// ---------------------------------------------------------------------------
// IQ4_XS, Q/reference/iq4_xs.rs:47-97; codebook Q/reference/iq_shared.rs:16-18.
// 136 B = f16 d, u16 scales_h, 4 B scales_l, 128 B nibble indices.  Unit = one
// 32-weight sub-block i: qs[16i..16i+16], interleaved nibbles.  Term:
// (d * (ls - 32)) * float(sum kvalues[idx] * a) * d_a.
struct FmtIQ4XS {
    static constexpr uint32_t BLOCK_BYTES = 136, BLOCK_COLS = 256, UNIT_COLS = 32;
    struct Lane {
        uint32_t i;
    };
    struct Act {
        uint32_t ev[4], od[4];
        float d_a;
    };
    struct Wt {
        u32x4 q;
        u32x2 hdr;
    };
    static __device__ __forceinline__ Lane lane_consts(uint32_t lane) { return Lane{lane & 7}; }
    static __device__ __forceinline__ void load_act(Act &a, const uint8_t *A, uint32_t u, bool valid,
                                                    const Lane &) {
        const uint8_t *blk = A + (size_t)u * Q8_BLOCK_BYTES;
        const u32x4 z = {0, 0, 0, 0};
        const u32x4 q0 = valid ? ld16(blk + 2) : z, q1 = valid ? ld16(blk + 18) : z;
        split_even_odd(q0, q1, a.ev, a.od);
        a.d_a = valid ? h2f(ld2(blk)) : 0.0f;
    }
    static __device__ __forceinline__ void load_w(Wt &w, const uint8_t *row, uint32_t u, bool valid,
                                                  const Lane &k) {
        const uint8_t *blk = row + (size_t)(u >> 3) * BLOCK_BYTES;
        const u32x4 z = {0, 0, 0, 0};
        const u32x2 z2 = {0, 0};
        w.hdr = valid ? ld8(blk) : z2;
        w.q = valid ? ld16(blk + 8 + 16 * k.i) : z;
    }
    // Four 4-bit indices (one per byte) -> four codebook bytes: two 8-entry byte
    // permutes, then a third permute picks the upper table where bit 3 is set.
    static __device__ __forceinline__ uint32_t lut4(uint32_t idx) {
        const uint32_t T0 = 0xBFAD9881u, T1 = 0xF6EADDCFu, T2 = 0x26190D01u, T3 = 0x71594535u;
        const uint32_t sel = idx & 0x07070707u;
        const uint32_t lo = __builtin_amdgcn_perm(T1, T0, sel);
        const uint32_t hi = __builtin_amdgcn_perm(T3, T2, sel);
        return __builtin_amdgcn_perm(hi, lo, 0x03020100u | ((idx >> 1) & 0x04040404u));
    }
    template <bool DUMP>
    static __device__ __forceinline__ float dot(const Wt &w, const Act &a, const Lane &k, int32_t *sums,
                                                uint32_t u, bool valid) {
        int p = 0;
        for (int i = 0; i < 4; i++) {
            p = sdot4(lut4(w.q[i] & 0x0F0F0F0Fu), a.ev[i], p);
            p = sdot4(lut4((w.q[i] >> 4) & 0x0F0F0F0Fu), a.od[i], p);
        }
        if (DUMP && valid) sums[u] = p;
        // unpack_sub_scale, iq4_xs.rs:47-53
        const uint32_t ls_low = (w.hdr[1] >> (4 * k.i)) & 0x0F;
        const uint32_t ls_high = ((w.hdr[0] >> 16) >> (2 * k.i)) & 0x03;
        const int ls = (int)(ls_low | (ls_high << 4)) - 32;
        const float scale = h2f(w.hdr[0] & 0xFFFF) * (float)ls;  // iq4_xs.rs:81
        return scale * (float)p * a.d_a;
    }
};

}  // namespace oxq
