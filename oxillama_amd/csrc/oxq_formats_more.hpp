// Lane work of the Q8_0-activation GEMV for the GGUF formats beyond the first five: Q4_1, Q5_0,
// Q5_1, Q8_1, IQ4_NL (32-weight blocks) and Q2_K, Q3_K, Q5_K (256-weight super-blocks).  Same
// contract as oxq_formats.hpp: a lane owns one unit of a row per step, keeps the activation
// bytes of its unit in registers, forms exact int32 group sums with v_dot4 and one fp32 term per
// group.  Byte layouts and formulas follow the reference's decoders (Q/reference/ =
// crates/oxillama-quant/src/reference in the reference tree), cited per format.
//
// Integer groups (the unit of the bit-exact check): 32 weights for the block formats and Q5_K,
// 16 weights for Q2_K and Q3_K.
#pragma once
#include "oxq_formats.hpp"

namespace oxq {

// Sum of the 32 int8 values of an activation block.
__device__ __forceinline__ int act_sum32(const u32x4 &q0, const u32x4 &q1) {
    int s = 0;
    for (int i = 0; i < 4; i++) {
        s = sdot4(q0[i], 0x01010101u, s);
        s = sdot4(q1[i], 0x01010101u, s);
    }
    return s;
}

// Bits 0..3 of x -> bit 0 of bytes 0..3 (x < 16): x * (1 + 2^7 + 2^14 + 2^21) puts bit j at
// position 8j, among others, and the mask keeps those four.
__device__ __forceinline__ uint32_t spread4(uint32_t x) {
    return (uint32_t)__umul24(x, 0x00204081u) & 0x01010101u;
}

// ---------------------------------------------------------------------------
// Q4_1, Q/reference/q4_1.rs:37-46.  20 B = f16 d, f16 m, 16 B nibbles; byte i holds weights 2i
// (low) and 2i+1 (high); w = d * nibble + m.  sum w a = d * sum(nibble a) + m * sum a.
struct FmtQ4_1 {
    static constexpr uint32_t BLOCK_BYTES = 20, BLOCK_COLS = 32, UNIT_COLS = 32;
    static constexpr uint32_t TYPE_ID = OXQ_TYPE_Q4_1;
    static constexpr uint32_t TWO_ROW_BATCH_BYTES = 3400;
    struct Lane {};
    struct Act {
        uint32_t ev[4], od[4];
        float d_a, b;  // b = d_a * sum(q_a)
    };
    struct Wt {
        u32x4 q;
        uint32_t dm;
    };
    static __device__ __forceinline__ Lane lane_consts(uint32_t) { return Lane{}; }
    template <class SRC>
    static __device__ __forceinline__ void load_act(Act &a, const SRC &src, uint32_t u, bool valid, const Lane &) {
        u32x4 q0, q1;
        uint32_t dbits;
        src.block(u, q0, q1, dbits);
        split_even_odd(q0, q1, a.ev, a.od);
        a.d_a = valid ? h2f(dbits) : 0.0f;
        a.b = a.d_a * (float)act_sum32(q0, q1);
    }
    static __device__ __forceinline__ void load_w(Wt &w, const uint8_t *row, uint32_t u, const Lane &) {
        const uint8_t *blk = row + (size_t)u * BLOCK_BYTES;
        w.dm = ld4(blk);
        w.q = ld16(blk + 4);
    }
    template <bool DUMP>
    static __device__ __forceinline__ float dot(const Wt &w, const Act &a, const Lane &, int32_t *sums, uint32_t u,
                                                bool valid) {
        int p = 0;
        for (int i = 0; i < 4; i++) {
            p = sdot4(w.q[i] & 0x0F0F0F0Fu, a.ev[i], p);
            p = sdot4((w.q[i] >> 4) & 0x0F0F0F0Fu, a.od[i], p);
        }
        if (DUMP && valid) sums[u] = p;
        return fmaf(h2f(w.dm & 0xFFFF) * a.d_a, (float)p, h2f(w.dm >> 16) * a.b);
    }
};

// ---------------------------------------------------------------------------
// Q5_0, Q/reference/q5_0.rs:39-55.  22 B = f16 d, u32 qh, 16 B nibbles; byte i holds the low four
// bits of weights i (low nibble) and i+16 (high nibble), bit i / i+16 of qh the fifth;
// w = d * (q5 - 16).  The fifth bits are spread to one per byte and merged into the nibble dword.
struct FmtQ5_0 {
    static constexpr uint32_t BLOCK_BYTES = 22, BLOCK_COLS = 32, UNIT_COLS = 32;
    static constexpr uint32_t TYPE_ID = OXQ_TYPE_Q5_0;
    static constexpr uint32_t TWO_ROW_BATCH_BYTES = 3400;
    struct Lane {};
    struct Act {
        u32x4 q0, q1;
        float d_a;
        int nasum16;  // -16 * sum(q_a)
    };
    // 22-byte blocks: three aligned loads cover a block exactly.  On a dword boundary: bytes 0..15, 16..19,
    // 20..21; two bytes off: bytes 2..17, 18..21 and the 2 bytes 0..1 (d).  dot() shifts the first form by 16 bits.
    struct Wt {
        u32x4 q;
        uint32_t q4, x, off;
    };
    static __device__ __forceinline__ Lane lane_consts(uint32_t) { return Lane{}; }
    template <class SRC>
    static __device__ __forceinline__ void load_act(Act &a, const SRC &src, uint32_t u, bool valid, const Lane &) {
        uint32_t dbits;
        src.block(u, a.q0, a.q1, dbits);
        a.d_a = valid ? h2f(dbits) : 0.0f;
        a.nasum16 = -16 * act_sum32(a.q0, a.q1);
    }
    static __device__ __forceinline__ void load_w(Wt &w, const uint8_t *row, uint32_t u, const Lane &) {
        const uint8_t *blk = row + (size_t)u * BLOCK_BYTES;
        w.off = (uint32_t)(reinterpret_cast<uintptr_t>(blk) & 2);
        const uint8_t *base = blk + w.off;
        w.q = *reinterpret_cast<const u32x4 *>(base);
        w.q4 = *reinterpret_cast<const uint32_t *>(base + 16);
        w.x = ld2(w.off ? blk : blk + 20);
    }
    // Exact sum of q5 * a over the block, q5 in 0..31, starting from `start`.
    static __device__ __forceinline__ int dot5(const u32x4 &q, uint32_t qh, const u32x4 &a0, const u32x4 &a1, int start) {
        int p = start;
        for (int i = 0; i < 4; i++) {
            const uint32_t lo = (q[i] & 0x0F0F0F0Fu) | (spread4((qh >> (4 * i)) & 0xFu) << 4);
            const uint32_t hi = ((q[i] >> 4) & 0x0F0F0F0Fu) | (spread4((qh >> (16 + 4 * i)) & 0xFu) << 4);
            p = sdot4(lo, a0[i], p);
            p = sdot4(hi, a1[i], p);
        }
        return p;
    }
    template <bool DUMP>
    static __device__ __forceinline__ float dot(const Wt &w, const Act &a, const Lane &, int32_t *sums, uint32_t u,
                                                bool valid) {
        const uint32_t sh = w.off ? 0u : 16u;
        const uint32_t dw[6] = {w.q[0], w.q[1], w.q[2], w.q[3], w.q4, w.x};
        const uint32_t qh = __builtin_amdgcn_alignbit(dw[1], dw[0], sh);
        u32x4 q;
        for (int i = 0; i < 4; i++) q[i] = __builtin_amdgcn_alignbit(dw[i + 2], dw[i + 1], sh);
        const int p = dot5(q, qh, a.q0, a.q1, a.nasum16);
        if (DUMP && valid) sums[u] = p;
        return (h2f(w.off ? w.x : (w.q[0] & 0xFFFFu)) * a.d_a) * (float)p;
    }
};

// ---------------------------------------------------------------------------
// Q5_1, Q/reference/q5_1.rs:38-56.  24 B = f16 d, f16 m, u32 qh, 16 B nibbles (as Q5_0);
// w = d * q5 + m.
struct FmtQ5_1 {
    static constexpr uint32_t BLOCK_BYTES = 24, BLOCK_COLS = 32, UNIT_COLS = 32;
    static constexpr uint32_t TYPE_ID = OXQ_TYPE_Q5_1;
    static constexpr uint32_t TWO_ROW_BATCH_BYTES = 3400;
    struct Lane {};
    struct Act {
        u32x4 q0, q1;
        float d_a, b;  // b = d_a * sum(q_a)
    };
    struct Wt {
        u32x4 q;
        u32x2 hdr;  // d | m << 16, qh
    };
    static __device__ __forceinline__ Lane lane_consts(uint32_t) { return Lane{}; }
    template <class SRC>
    static __device__ __forceinline__ void load_act(Act &a, const SRC &src, uint32_t u, bool valid, const Lane &) {
        uint32_t dbits;
        src.block(u, a.q0, a.q1, dbits);
        a.d_a = valid ? h2f(dbits) : 0.0f;
        a.b = a.d_a * (float)act_sum32(a.q0, a.q1);
    }
    static __device__ __forceinline__ void load_w(Wt &w, const uint8_t *row, uint32_t u, const Lane &) {
        const uint8_t *blk = row + (size_t)u * BLOCK_BYTES;
        w.hdr = ld8(blk);
        w.q = ld16(blk + 8);
    }
    template <bool DUMP>
    static __device__ __forceinline__ float dot(const Wt &w, const Act &a, const Lane &, int32_t *sums, uint32_t u,
                                                bool valid) {
        const int p = FmtQ5_0::dot5(w.q, w.hdr[1], a.q0, a.q1, 0);
        if (DUMP && valid) sums[u] = p;
        return fmaf(h2f(w.hdr[0] & 0xFFFF) * a.d_a, (float)p, h2f(w.hdr[0] >> 16) * a.b);
    }
};

// ---------------------------------------------------------------------------
// Q8_1, Q/reference/q8_1.rs:36-42.  36 B = f16 d, f16 s (d * sum q, unused), 32 x i8; w = d * q.
struct FmtQ8_1 {
    static constexpr uint32_t BLOCK_BYTES = 36, BLOCK_COLS = 32, UNIT_COLS = 32;
    static constexpr uint32_t TYPE_ID = OXQ_TYPE_Q8_1;
    static constexpr uint32_t TWO_ROW_BATCH_BYTES = 3400;
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
    template <class SRC>
    static __device__ __forceinline__ void load_act(Act &a, const SRC &src, uint32_t u, bool valid, const Lane &) {
        uint32_t dbits;
        src.block(u, a.q0, a.q1, dbits);
        a.d_a = valid ? h2f(dbits) : 0.0f;
    }
    static __device__ __forceinline__ void load_w(Wt &w, const uint8_t *row, uint32_t u, const Lane &) {
        const uint8_t *blk = row + (size_t)u * BLOCK_BYTES;
        w.d = ld2(blk);
        w.q0 = ld16(blk + 4);
        w.q1 = ld16(blk + 20);
    }
    template <bool DUMP>
    static __device__ __forceinline__ float dot(const Wt &w, const Act &a, const Lane &, int32_t *sums, uint32_t u,
                                                bool valid) {
        int p = 0;
        for (int i = 0; i < 4; i++) {
            p = sdot4(w.q0[i], a.q0[i], p);
            p = sdot4(w.q1[i], a.q1[i], p);
        }
        if (DUMP && valid) sums[u] = p;
        return (h2f(w.d) * a.d_a) * (float)p;
    }
};

// ---------------------------------------------------------------------------
// IQ4_NL, Q/reference/iq4_nl.rs:43-51.  18 B = f16 d, 16 B nibble indices into the codebook
// (Q/reference/iq_shared.rs:16-18); byte i holds weights 2i (low) and 2i+1 (high); w = d * kv[idx].
struct FmtIQ4NL {
    static constexpr uint32_t BLOCK_BYTES = 18, BLOCK_COLS = 32, UNIT_COLS = 32;
    static constexpr uint32_t TYPE_ID = OXQ_TYPE_IQ4_NL;
    static constexpr uint32_t TWO_ROW_BATCH_BYTES = 3400;
    struct Lane {};
    struct Act {
        uint32_t ev[4], od[4];
        float d_a;
    };
    // loaded as FmtQ4_0's blocks: one dword-aligned 16-byte load (bytes 0..15 of a block on a dword
    // boundary, bytes 2..17 of one two bytes off) and one 2-byte load for the rest
    struct Wt {
        u32x4 q;
        uint32_t x, off;
    };
    static __device__ __forceinline__ Lane lane_consts(uint32_t) { return Lane{}; }
    template <class SRC>
    static __device__ __forceinline__ void load_act(Act &a, const SRC &src, uint32_t u, bool valid, const Lane &) {
        u32x4 q0, q1;
        uint32_t dbits;
        src.block(u, q0, q1, dbits);
        split_even_odd(q0, q1, a.ev, a.od);
        a.d_a = valid ? h2f(dbits) : 0.0f;
    }
    static __device__ __forceinline__ void load_w(Wt &w, const uint8_t *row, uint32_t u, const Lane &) {
        const uint8_t *blk = row + (size_t)u * BLOCK_BYTES;
        w.off = (uint32_t)(reinterpret_cast<uintptr_t>(blk) & 2);
        w.q = *reinterpret_cast<const u32x4 *>(blk + w.off);
        w.x = ld2(w.off ? blk : blk + 16);
    }
    template <bool DUMP>
    static __device__ __forceinline__ float dot(const Wt &w, const Act &a, const Lane &, int32_t *sums, uint32_t u,
                                                bool valid) {
        const uint32_t sh = w.off ? 0u : 16u;
        const uint32_t dw[5] = {w.q[0], w.q[1], w.q[2], w.q[3], w.x};
        int p = 0;
        for (int i = 0; i < 4; i++) {
            const uint32_t q = __builtin_amdgcn_alignbit(dw[i + 1], dw[i], sh);
            p = sdot4(FmtIQ4XS::lut4(q & 0x0F0F0F0Fu), a.ev[i], p);
            p = sdot4(FmtIQ4XS::lut4((q >> 4) & 0x0F0F0F0Fu), a.od[i], p);
        }
        if (DUMP && valid) sums[u] = p;
        return (h2f(w.off ? w.x : (w.q[0] & 0xFFFFu)) * a.d_a) * (float)p;
    }
};

// ---------------------------------------------------------------------------
// Q5_K, Q/reference/q5_k.rs:27-102,270-345.  176 B = f16 d, f16 dmin, 12 B packed 6-bit scales /
// mins (as Q4_K), 32 B qh, 128 B nibbles.  Unit = 64-weight group g: qs[32g..32g+32] low nibbles
// = sub-block 2g, high nibbles = sub-block 2g+1; the fifth bit of weight l is bit g (low) / g+4
// (high) of qh[l].  Term per sub-block: (d*sc*sum(q5 a) - dmin*mn*sum a) * d_a.
struct FmtQ5K {
    static constexpr uint32_t BLOCK_BYTES = 176, BLOCK_COLS = 256, UNIT_COLS = 64;
    static constexpr uint32_t TYPE_ID = OXQ_TYPE_Q5_K;
    // measured: two rows per batch beat one at both 14336 x 4096 and 4096 x 14336 (11.1 -> 10.4-10.8 us)
    static constexpr uint32_t TWO_ROW_BATCH_BYTES = 4000;
    using Lane = FmtQ4K::Lane;
    struct Act {
        u32x4 lo0, lo1, hi0, hi1;
        float a_lo, a_hi, b_lo, b_hi;  // d_a and d_a * sum(q_a) of the two activation blocks
    };
    struct Wt {
        u32x4 hdr, h0, h1, q0, q1;
    };
    static __device__ __forceinline__ Lane lane_consts(uint32_t lane) { return FmtQ4K::lane_consts(lane); }
    template <class SRC>
    static __device__ __forceinline__ void load_act(Act &a, const SRC &src, uint32_t u, bool valid, const Lane &k) {
        uint32_t dlo_bits, dhi_bits;
        src.block(8 * (u >> 2) + 2 * k.g, a.lo0, a.lo1, dlo_bits);
        src.block(8 * (u >> 2) + 2 * k.g + 1, a.hi0, a.hi1, dhi_bits);
        const float dlo = h2f(dlo_bits), dhi = h2f(dhi_bits);
        a.a_lo = valid ? dlo : 0.0f;
        a.a_hi = valid ? dhi : 0.0f;
        a.b_lo = a.a_lo * (float)act_sum32(a.lo0, a.lo1);
        a.b_hi = a.a_hi * (float)act_sum32(a.hi0, a.hi1);
    }
    static __device__ __forceinline__ void load_w(Wt &w, const uint8_t *row, uint32_t u, const Lane &k) {
        const uint8_t *blk = row + (size_t)(u >> 2) * BLOCK_BYTES;
        w.hdr = ld16(blk);
        w.h0 = ld16(blk + 16);
        w.h1 = ld16(blk + 32);
        w.q0 = ld16(blk + 48 + 32 * k.g);
        w.q1 = ld16(blk + 64 + 32 * k.g);
    }
    template <bool DUMP>
    static __device__ __forceinline__ float dot(const Wt &w, const Act &a, const Lane &k, int32_t *sums, uint32_t u,
                                                bool valid) {
        int plo = 0, phi = 0;
        for (int i = 0; i < 4; i++) {
            const uint32_t b0 = w.h0[i] >> k.g, b1 = w.h1[i] >> k.g;
            plo = sdot4((w.q0[i] & 0x0F0F0F0Fu) | ((b0 & 0x01010101u) << 4), a.lo0[i], plo);
            phi = sdot4(((w.q0[i] >> 4) & 0x0F0F0F0Fu) | (b0 & 0x10101010u), a.hi0[i], phi);
            plo = sdot4((w.q1[i] & 0x0F0F0F0Fu) | ((b1 & 0x01010101u) << 4), a.lo1[i], plo);
            phi = sdot4(((w.q1[i] >> 4) & 0x0F0F0F0Fu) | (b1 & 0x10101010u), a.hi1[i], phi);
        }
        if (DUMP && valid) {
            sums[2 * u] = plo;
            sums[2 * u + 1] = phi;
        }
        // scales / mins of sub-blocks 2g, 2g+1 (decode_scales_mins, q5_k.rs:27-49; as Q4_K)
        const uint32_t sa = w.hdr[1] >> k.sh, sb = w.hdr[2] >> k.sh, sc3 = w.hdr[3] >> k.sh;
        const uint32_t x = k.upper ? sc3 : sa, y = k.upper ? (sc3 >> 4) : sb;
        const uint32_t m1 = k.upper ? 0x0F0Fu : 0x3F3Fu, m2 = k.upper ? 0x3030u : 0u;
        const uint32_t sc2 = (x & m1) | ((sa >> 2) & m2);
        const uint32_t mn2 = (y & m1) | ((sb >> 2) & m2);
        const float d = h2f(w.hdr[0] & 0xFFFF), dmin = h2f(w.hdr[0] >> 16);
        // |sum| <= 32 * 31 * 128 < 2^17, times a 6-bit scale < 2^23: exact
        float su = a.a_lo * (float)mul24(plo, (int)(sc2 & 0xFF));
        su = fmaf(a.a_hi, (float)mul24(phi, (int)((sc2 >> 8) & 0xFF)), su);
        float sv = a.b_lo * (float)(mn2 & 0xFF);
        sv = fmaf(a.b_hi, (float)((mn2 >> 8) & 0xFF), sv);
        return fmaf(d, su, -(dmin * sv));
    }
};

// Activation side shared by Q2_K and Q3_K.  Unit = (group n, half hf) of a super-block: 16 bytes of
// qs give four 16-weight sub-blocks at columns 128n + 32j + 16hf (j = 0..3), i.e. half hf of
// activation blocks 8b + 4n + j.
struct Act16x4 {
    u32x4 q[4];
    float d_a[4];
    int asum[4];  // sum of the 16 activation bytes
};
template <class SRC>
__device__ __forceinline__ void load_act16x4(Act16x4 &a, const SRC &src, uint32_t u, bool valid, uint32_t n,
                                             uint32_t hf) {
    const u32x4 z = {0, 0, 0, 0};
    for (int j = 0; j < 4; j++) {
        u32x4 q0, q1;
        uint32_t dbits;
        src.block(8 * (u >> 2) + 4 * n + j, q0, q1, dbits);
        const u32x4 q = hf ? q1 : q0;
        a.q[j] = valid ? q : z;
        a.d_a[j] = valid ? h2f(dbits) : 0.0f;
        int s = 0;
        for (int i = 0; i < 4; i++) s = sdot4(a.q[j][i], 0x01010101u, s);
        a.asum[j] = s;
    }
}

// ---------------------------------------------------------------------------
// Q2_K, Q/reference/q2_k.rs:41-80,224-292.  84 B = 16 scale bytes (low nibble scale, high nibble
// min), 64 B of 2-bit quants, f16 d, f16 dmin.  Sub-block is = 8n + 2j + hf takes bits 2j..2j+1
// of qs[32n + 16hf + l]; term (d*sc*sum(q a) - dmin*mn*sum a) * d_a per 16 weights.
struct FmtQ2K {
    static constexpr uint32_t BLOCK_BYTES = 84, BLOCK_COLS = 256, UNIT_COLS = 64;
    static constexpr uint32_t TYPE_ID = OXQ_TYPE_Q2_K;
    static constexpr uint32_t TWO_ROW_BATCH_BYTES = 4000;  // measured: 9.5-9.9 -> 8.4-8.8 us with two rows per batch
    struct Lane {
        uint32_t n, hf;
    };
    using Act = Act16x4;
    struct Wt {
        u32x4 q;
        u32x2 sc;
        uint32_t dd;
    };
    static __device__ __forceinline__ Lane lane_consts(uint32_t lane) { return Lane{(lane >> 1) & 1, lane & 1}; }
    template <class SRC>
    static __device__ __forceinline__ void load_act(Act &a, const SRC &src, uint32_t u, bool valid, const Lane &k) {
        load_act16x4(a, src, u, valid, k.n, k.hf);
    }
    static __device__ __forceinline__ void load_w(Wt &w, const uint8_t *row, uint32_t u, const Lane &k) {
        const uint8_t *blk = row + (size_t)(u >> 2) * BLOCK_BYTES;
        w.sc = ld8(blk + 8 * k.n);
        w.q = ld16(blk + 16 + 32 * k.n + 16 * k.hf);
        w.dd = ld4(blk + 80);
    }
    template <bool DUMP>
    static __device__ __forceinline__ float dot(const Wt &w, const Act &a, const Lane &k, int32_t *sums, uint32_t u,
                                                bool valid) {
        int p[4] = {0, 0, 0, 0};
        for (int i = 0; i < 4; i++)
            for (int j = 0; j < 4; j++) p[j] = sdot4((w.q[i] >> (2 * j)) & 0x03030303u, a.q[j][i], p[j]);
        // scale byte 2j + hf of the group's eight
        const uint32_t s0 = w.sc[0] >> (8 * k.hf), s1 = w.sc[1] >> (8 * k.hf);
        const uint32_t sb[4] = {s0 & 0xFF, (s0 >> 16) & 0xFF, s1 & 0xFF, (s1 >> 16) & 0xFF};
        float su = 0.0f, sv = 0.0f;
        for (int j = 0; j < 4; j++) {
            // |sum| <= 16 * 3 * 128, times a 4-bit scale: exact
            su = fmaf(a.d_a[j], (float)mul24(p[j], (int)(sb[j] & 0x0F)), su);
            sv = fmaf(a.d_a[j], (float)mul24(a.asum[j], (int)(sb[j] >> 4)), sv);
            if (DUMP && valid) sums[16 * (u >> 2) + 8 * k.n + 2 * j + k.hf] = p[j];
        }
        return fmaf(h2f(w.dd & 0xFFFF), su, -(h2f(w.dd >> 16) * sv));
    }
};

// ---------------------------------------------------------------------------
// Q3_K, Q/reference/q3_k.rs:30-59,76-120,258-322.  110 B = 32 B hmask, 64 B of 2-bit quants, 12 B
// packed 6-bit scales (value - 32), f16 d.  Sub-block is = 8n + 2j + hf: q3 = (qs[32n + 16hf + l]
// >> 2j & 3) - (hmask[16hf + l] bit (4n + j) ? 0 : 4); term d * (sc - 32) * sum(q3 a) * d_a.
struct FmtQ3K {
    static constexpr uint32_t BLOCK_BYTES = 110, BLOCK_COLS = 256, UNIT_COLS = 64;
    static constexpr uint32_t TYPE_ID = OXQ_TYPE_Q3_K;
    // measured: 11.9-12.3 -> 10.8-11.0 us with two rows per batch and four waves per compute unit
    static constexpr uint32_t TWO_ROW_BATCH_BYTES = 4000;
    static constexpr uint32_t WAVES_PER_CU = 4;
    using Lane = FmtQ2K::Lane;
    using Act = Act16x4;
    struct Wt {
        u32x4 q, hm;
        u32x2 s01;
        uint32_t s2, d;
    };
    static __device__ __forceinline__ Lane lane_consts(uint32_t lane) { return FmtQ2K::lane_consts(lane); }
    template <class SRC>
    static __device__ __forceinline__ void load_act(Act &a, const SRC &src, uint32_t u, bool valid, const Lane &k) {
        load_act16x4(a, src, u, valid, k.n, k.hf);
    }
    static __device__ __forceinline__ void load_w(Wt &w, const uint8_t *row, uint32_t u, const Lane &k) {
        const uint8_t *blk = row + (size_t)(u >> 2) * BLOCK_BYTES;
        w.hm = ld16(blk + 16 * k.hf);
        w.q = ld16(blk + 32 + 32 * k.n + 16 * k.hf);
        w.s01 = ld8(blk + 96);
        w.s2 = ld4(blk + 104);
        w.d = ld2(blk + 108);
    }
    template <bool DUMP>
    static __device__ __forceinline__ float dot(const Wt &w, const Act &a, const Lane &k, int32_t *sums, uint32_t u,
                                                bool valid) {
        // sum (v - 4) a = sum v a - 4 sum a with v = q_lo | hbit << 2
        int p[4] = {-4 * a.asum[0], -4 * a.asum[1], -4 * a.asum[2], -4 * a.asum[3]};
        for (int i = 0; i < 4; i++) {
            const uint32_t hb = w.hm[i] >> (4 * k.n);
            for (int j = 0; j < 4; j++) {
                const uint32_t v = ((w.q[i] >> (2 * j)) & 0x03030303u) | (((hb >> j) & 0x01010101u) << 2);
                p[j] = sdot4(v, a.q[j][i], p[j]);
            }
        }
        // decode_scales (q3_k.rs:30-59) for index 8n + kk, kk = 2j + hf: n = 0: s[kk] & 63;
        // n = 1: nibble (kk >> 2) of s[8 + (kk & 3)] | (s[kk] >> 6) << 4.
        float t = 0.0f;
        for (int j = 0; j < 4; j++) {
            const uint32_t sh = 8 * (2 * (j & 1) + k.hf);
            const uint32_t byte = ((j < 2 ? w.s01[0] : w.s01[1]) >> sh) & 0xFF;
            const uint32_t hi = ((w.s2 >> (sh + 4 * (j >> 1))) & 0x0F) | ((byte >> 6) << 4);
            const int sc = (int)(k.n ? hi : (byte & 0x3F)) - 32;
            // |sum| <= 16 * 4 * 128 = 2^13, |sc| <= 32: exact
            t = fmaf(a.d_a[j], (float)mul24(p[j], sc), t);
            if (DUMP && valid) sums[16 * (u >> 2) + 8 * k.n + 2 * j + k.hf] = p[j];
        }
        return h2f(w.d) * t;
    }
};

}  // namespace oxq
