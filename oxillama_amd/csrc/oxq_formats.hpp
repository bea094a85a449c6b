// Per-format lane work for the Q8_0-activation GEMV on gfx950.
//
// A row of n_cols weights is cut into "units"; lane l of a wave owns unit
// 64*step + l.  For each format this file says which raw GGUF bytes the lane
// loads for its unit (Wt), which Q8_0 activation bytes and derived constants it
// keeps in registers for every row (Act), and how the exact int32 group sums
// and the fp32 contribution are formed from them.  Byte layouts follow the
// reference decoders cited below (Q/ = crates/oxillama-quant/src in the
// reference tree).
//
// Integer groups (the unit of the bit-exact check): 32 weights = one Q8_0
// activation block for Q4_0 / Q8_0 / Q4_K / IQ4_XS, 16 weights for Q6_K.
//
// Loads are unconditional: a lane past the end of the row (`valid` false) reads
// the row's last unit instead and carries all-zero activation constants, so it
// contributes exactly 0 without any divergent control flow.
//
// fp32 form.  With I = integer group sum, the reference's fused rows compute
// (d*sc*I - dmin*mn*S) * d_a per group (Q/simd/avx2/q4_k.rs:329).  d*sc, dmin*mn
// and the products sc*I, mn*S are exact in fp32 (11-bit f16 significand times a
// 6..8-bit integer; |sc*I| < 2^24), so d*float(sc*I) rounds exactly as
// (d*sc)*float(I) does.  The kernels use that to do the scale multiplications in
// integer arithmetic, and they accumulate the groups of one unit with fused
// multiply-adds before the cross-lane sum; only the accumulation order and the
// placement of roundings differ from the reference, within the 1e-5*|y|inf bar.
#pragma once
#include "../../include/oxq.h"
#include "oxq_device.hpp"

namespace oxq {

constexpr uint32_t Q8_BLOCK_BYTES = 34;  // Q/traits.rs:12: f16 d + 32 x i8

// v_mul_i32_i24: exact product of two values that fit in 24 signed bits.
__device__ __forceinline__ int mul24(int a, int b) { return __mul24(a, b); }

// Where a wave takes its activations from.  Both sources hand out one Q8_0 block as it sits
// in the reference's acts_q8 buffer: 32 int8 (two 16-byte halves) and the f16 scale bits.
//  * ActQ8: the blocks were quantized beforehand (oxq_quantize_q8_0_dev) and are read.
//  * ActF32: fp32 activations; every work group first quantizes the vector into LDS with the
//    arithmetic of encode_q8_0_block (crates/oxillama-quant/src/quantize.rs:190-210) -- the
//    same bytes, without a separate quantize launch (QuantKernel::gemv takes fp32 input,
//    crates/oxillama-quant/src/traits.rs:39-44) -- and its waves read the blocks from there.
struct ActQ8 {
    const uint8_t *A;
    static __device__ __forceinline__ ActQ8 make(const void *p, uint32_t) { return ActQ8{static_cast<const uint8_t *>(p)}; }
    __device__ __forceinline__ void block(uint32_t b, u32x4 &q0, u32x4 &q1, uint32_t &dbits) const {
        const uint8_t *blk = A + (size_t)b * Q8_BLOCK_BYTES;
        q0 = ld16(blk + 2);
        q1 = ld16(blk + 18);
        dbits = ld2(blk);
    }
};
// The same blocks for a row that ends inside a block: the reference skips the columns past n_cols
// (crates/oxillama-quant/src/reference/q4_k.rs:307-321, traits.rs:150-166), which is a dot product
// with zero activations there, so the payload bytes of those columns read as zero.
struct ActQ8Tail {
    const uint8_t *A;
    uint32_t n_cols;
    // Bytes off..off+3 of a block of which only the first `rem` columns exist.
    static __device__ __forceinline__ uint32_t tail_mask(uint32_t rem, uint32_t off) {
        const uint32_t keep = rem > off ? min(rem - off, 4u) : 0u;
        return keep >= 4 ? 0xFFFFFFFFu : (1u << (8 * keep)) - 1u;
    }
    __device__ __forceinline__ void block(uint32_t b, u32x4 &q0, u32x4 &q1, uint32_t &dbits) const {
        ActQ8{A}.block(b, q0, q1, dbits);
        if (32 * b + 32 > n_cols) {
            const uint32_t rem = n_cols > 32 * b ? n_cols - 32 * b : 0;
            for (int i = 0; i < 4; i++) {
                q0[i] &= tail_mask(rem, 4 * i);
                q1[i] &= tail_mask(rem, 16 + 4 * i);
            }
        }
    }
};
struct ActF32 {
    const float *X;
    static __device__ __forceinline__ ActF32 make(const void *p, uint32_t) { return ActF32{static_cast<const float *>(p)}; }
};
// The blocks ActF32 stands for, once the work group has quantized them into LDS
// (quantize_to_lds): 32 payload bytes per block, 32-byte aligned, and the f16 scales apart.
struct ActLds {
    const u32x4 *q;     // [n_blocks][2]
    const uint16_t *d;  // [n_blocks]
    __device__ __forceinline__ void block(uint32_t b, u32x4 &q0, u32x4 &q1, uint32_t &dbits) const {
        q0 = q[2 * b];
        q1 = q[2 * b + 1];
        dbits = d[b];
    }
};

// All 256 threads of a work group quantize n_blocks * 32 floats into LDS: eight lanes per
// block, four floats per lane, exactly as quantize_q8_0_kernel does.
__device__ __forceinline__ void quantize_to_lds(const float *__restrict__ x, uint32_t n_blocks, uint32_t n_cols,
                                                uint32_t *lds_q, uint16_t *lds_d) {
    const uint32_t j = threadIdx.x & 7;
    for (uint32_t base = 0; base < n_blocks; base += 32) {
        const uint32_t blk = base + (threadIdx.x >> 3);
        const bool valid = blk < n_blocks;
        float v[4] = {0.0f, 0.0f, 0.0f, 0.0f};
        const uint32_t col = blk * 32 + 4 * j;
        if (valid && col + 4 <= n_cols) {
            const u32x4 raw = *reinterpret_cast<const u32x4 *>(x + col);
            for (int i = 0; i < 4; i++) {
                const uint32_t bits = raw[i];  // copy out first: bit_cast must not see the vector element lvalue
                v[i] = __builtin_bit_cast(float, bits);
            }
        } else if (valid) {  // the row ends inside these four: the columns past it count as 0.0
            for (int i = 0; i < 4; i++)
                if (col + i < n_cols) v[i] = x[col + i];
        }
        float m = 0.0f;
        for (int i = 0; i < 4; i++) m = fmaxf(m, fabsf(v[i]));
        m = fmaxf(m, dpp_f<0xB1>(m));
        m = fmaxf(m, dpp_f<0x4E>(m));
        m = fmaxf(m, __shfl_xor(m, 4, 64));  // max is exact in any order (quantize.rs:194)
        const float d = m / 127.0f;                      // quantize.rs:197
        const float id = (d != 0.0f) ? 1.0f / d : 0.0f;  // quantize.rs:198
        uint32_t packed = 0;
        for (int i = 0; i < 4; i++) {
            int q = (int)roundf(v[i] * id);  // quantize.rs:206 (round half away from zero)
            q = q < -128 ? -128 : (q > 127 ? 127 : q);
            packed |= ((uint32_t)q & 0xFFu) << (8 * i);
        }
        if (valid) {
            lds_q[blk * 8 + j] = packed;
            if (j == 0) lds_d[blk] = (uint16_t)f2h(d);  // quantize.rs:201
        }
    }
}

// ---------------------------------------------------------------------------
// Q4_K, Q/reference/q4_k.rs:27-99,218-333.  144 B = d, dmin (f16), 12 B packed
// 6-bit scales/mins, 128 B nibbles.  Unit = one 64-weight group g (0..3) of a
// super-block: qs[32g..32g+32], low nibbles = sub-block 2g, high nibbles =
// sub-block 2g+1, against activation blocks 8b+2g and 8b+2g+1.  Four lanes per
// super-block; the 16-byte header is read by each of them (same cache line).
struct FmtQ4K {
    static constexpr uint32_t BLOCK_BYTES = 144, BLOCK_COLS = 256, UNIT_COLS = 64;
    static constexpr uint32_t TYPE_ID = OXQ_TYPE_Q4_K;
    static constexpr uint32_t TWO_ROW_BATCH_BYTES = 3400;  // two rows per batch up to this slice of a row per wave
    struct Lane {
        uint32_t g, sh;
        bool upper;
    };
    struct Act {
        u32x4 lo0, lo1, hi0, hi1;
        float a_lo, a_hi16;  // d_a of the low-nibble block; d_a / 16 of the high-nibble block
        float b_lo, b_hi;    // d_a * sum(q_a)
        int s_hi128;         // 128 * sum(q_a) of the high-nibble block
    };
    struct Wt {
        u32x4 hdr, q0, q1;
    };
    static __device__ __forceinline__ Lane lane_consts(uint32_t lane) {
        Lane k;
        k.g = lane & 3;
        k.sh = (k.g & 1) * 16;
        k.upper = k.g >= 2;
        return k;
    }
    template <class SRC>
    static __device__ __forceinline__ void load_act(Act &a, const SRC &src, uint32_t u, bool valid, const Lane &k) {
        uint32_t dlo_bits, dhi_bits;
        src.block(8 * (u >> 2) + 2 * k.g, a.lo0, a.lo1, dlo_bits);
        src.block(8 * (u >> 2) + 2 * k.g + 1, a.hi0, a.hi1, dhi_bits);
        int slo = 0, shi = 0;
        for (int i = 0; i < 4; i++) {
            slo = sdot4(a.lo0[i], 0x01010101u, slo);
            slo = sdot4(a.lo1[i], 0x01010101u, slo);
            shi = sdot4(a.hi0[i], 0x01010101u, shi);
            shi = sdot4(a.hi1[i], 0x01010101u, shi);
        }
        const float dlo = h2f(dlo_bits), dhi = h2f(dhi_bits);
        a.a_lo = valid ? dlo : 0.0f;
        a.a_hi16 = valid ? dhi * 0.0625f : 0.0f;  // exact
        a.b_lo = valid ? dlo * (float)slo : 0.0f;
        a.b_hi = valid ? dhi * (float)shi : 0.0f;
        a.s_hi128 = 128 * shi;
    }
    static __device__ __forceinline__ void load_w(Wt &w, const uint8_t *row, uint32_t u, const Lane &k) {
        const uint8_t *blk = row + (size_t)(u >> 2) * BLOCK_BYTES;
        w.hdr = ld16(blk);
        w.q0 = ld16(blk + 16 + 32 * k.g);
        w.q1 = ld16(blk + 32 + 32 * k.g);
    }
    template <bool DUMP>
    static __device__ __forceinline__ float dot(const Wt &w, const Act &a, const Lane &k, int32_t *sums,
                                                uint32_t u, bool valid) {
        // Low nibbles: q & 0x0F.  High nibbles stay in place: (q & 0xF0) ^ 0x80 read as a signed byte is
        // 16 * (n - 8), so the dot product is 16 * (sum n*a - 8 * sum a); adding 128 * sum a gives
        // 16 * phi exactly, one operation per dword instead of a shift and a mask.
        int plo = 0, phi16 = a.s_hi128;
        for (int i = 0; i < 4; i++) {
            plo = sdot4(w.q0[i] & 0x0F0F0F0Fu, a.lo0[i], plo);
            phi16 = sdot4((w.q0[i] & 0xF0F0F0F0u) ^ 0x80808080u, a.hi0[i], phi16);
            plo = sdot4(w.q1[i] & 0x0F0F0F0Fu, a.lo1[i], plo);
            phi16 = sdot4((w.q1[i] & 0xF0F0F0F0u) ^ 0x80808080u, a.hi1[i], phi16);
        }
        if (DUMP && valid) {
            sums[2 * u] = plo;
            sums[2 * u + 1] = phi16 >> 4;
        }
        // 6-bit scales / mins of sub-blocks 2g, 2g+1 as byte pairs (decode_scales_mins,
        // q4_k.rs:27-49): j < 4: sc = s[j] & 63, mn = s[j+4] & 63; j >= 4: sc = (s[j+4] & 15) |
        // (s[j-4] >> 6) << 4, mn = (s[j+4] >> 4) | (s[j] >> 6) << 4.
        const uint32_t sa = w.hdr[1] >> k.sh, sb = w.hdr[2] >> k.sh, sc3 = w.hdr[3] >> k.sh;
        const uint32_t x = k.upper ? sc3 : sa, y = k.upper ? (sc3 >> 4) : sb;
        const uint32_t m1 = k.upper ? 0x0F0Fu : 0x3F3Fu, m2 = k.upper ? 0x3030u : 0u;
        const uint32_t sc2 = (x & m1) | ((sa >> 2) & m2);
        const uint32_t mn2 = (y & m1) | ((sb >> 2) & m2);
        const float d = h2f(w.hdr[0] & 0xFFFF), dmin = h2f(w.hdr[0] >> 16);
        float su = a.a_lo * (float)mul24(plo, (int)(sc2 & 0xFF));
        // |16 phi| < 2^20 fits mul24; 16 * phi * sc is a multiple of 16 below 2^26: exact in fp32
        su = fmaf(a.a_hi16, (float)mul24(phi16, (int)((sc2 >> 8) & 0xFF)), su);
        float sv = a.b_lo * (float)(mn2 & 0xFF);
        sv = fmaf(a.b_hi, (float)((mn2 >> 8) & 0xFF), sv);
        return fmaf(d, su, -(dmin * sv));
    }
};

// ---------------------------------------------------------------------------
// Q6_K, Q/reference/q6_k.rs:39-72,246-351.  210 B = ql[128], qh[64], i8
// scales[16], f16 d.  Unit = (half hh, sixteen is) of a super-block: bytes
// ql[64hh+16is..+16], ql[64hh+32+16is..+16], qh[32hh+16is..+16] give four
// 16-weight sub-blocks at columns 128hh + 32j + 16is (j = 0..3), scale index
// 8hh + is + 2j, activation block 8b + 4hh + j bytes 16is..+16.
struct FmtQ6K {
    static constexpr uint32_t BLOCK_BYTES = 210, BLOCK_COLS = 256, UNIT_COLS = 64;
    static constexpr uint32_t TYPE_ID = OXQ_TYPE_Q6_K;
    // Measured on MI355X (4096 x 14336 and 128256 x 4096): four waves per compute unit with two rows per
    // batch beat eight waves with one (11.4 against 11.8 us, 73.6 against 76.6 us).
    static constexpr uint32_t TWO_ROW_BATCH_BYTES = 4000;
    static constexpr uint32_t WAVES_PER_CU = 4;
    struct Lane {
        uint32_t hh, is;
    };
    struct Act {
        u32x4 q[4];
        float d_a[4];
        int nasum32[4];  // -32 * sum of the 16 activation bytes
    };
    struct Wt {
        u32x4 ql0, ql1, qh;  // as loaded from the dword-aligned address at or below the lane's bytes
        u32x2 sc;
        uint32_t sc2;        // the dword after sc (needed when the block sits off a dword boundary)
        uint32_t d;
        uint32_t sh;         // bits by which the loaded dwords are off: 8 * (block address % 4)
    };
    static __device__ __forceinline__ Lane lane_consts(uint32_t lane) {
        Lane k;
        k.hh = (lane >> 1) & 1;
        k.is = lane & 1;
        return k;
    }
    template <int CTRL> static __device__ __forceinline__ uint32_t qp(uint32_t v) { return (uint32_t)dpp_i<CTRL>((int)v); }
    // 16 bytes that start `sh` bits into x: x holds the 16 bytes at the aligned address below, `next` the dword after
    static __device__ __forceinline__ u32x4 realign(const u32x4 x, uint32_t next, uint32_t sh) {
        u32x4 r;
        r[0] = __builtin_amdgcn_alignbit(x[1], x[0], sh);
        r[1] = __builtin_amdgcn_alignbit(x[2], x[1], sh);
        r[2] = __builtin_amdgcn_alignbit(x[3], x[2], sh);
        r[3] = __builtin_amdgcn_alignbit(next, x[3], sh);
        return r;
    }
    template <class SRC>
    static __device__ __forceinline__ void load_act(Act &a, const SRC &src, uint32_t u, bool valid, const Lane &k) {
        const u32x4 z = {0, 0, 0, 0};
        for (int j = 0; j < 4; j++) {
            u32x4 q0, q1;
            uint32_t dbits;
            src.block(8 * (u >> 2) + 4 * k.hh + j, q0, q1, dbits);
            const u32x4 q = k.is ? q1 : q0;
            a.q[j] = valid ? q : z;
            a.d_a[j] = valid ? h2f(dbits) : 0.0f;
            int s = 0;
            for (int i = 0; i < 4; i++) s = sdot4(a.q[j][i], 0x01010101u, s);
            a.nasum32[j] = -32 * s;
        }
    }
    static __device__ __forceinline__ void load_w(Wt &w, const uint8_t *row, uint32_t u, const Lane &k) {
        const uint8_t *blk = row + (size_t)(u >> 2) * BLOCK_BYTES;
        // A block is 210 bytes, so every other block sits two bytes off a dword boundary, and 16-byte loads
        // from such addresses cost a large part of the load bandwidth.  All loads therefore go to the
        // dword-aligned address at or below; the missing last bytes of a lane's piece are the first bytes of
        // the neighbouring lane's load (the pieces of a block are consecutive), fetched in dot() with DPP.
        // W is dword-aligned (checked by the host), so the two bytes below a block are inside the matrix.
        const uint32_t off = (uint32_t)(reinterpret_cast<uintptr_t>(blk) & 3);
        const uint8_t *base = blk - off;
        w.sh = 8 * off;
        w.ql0 = *reinterpret_cast<const u32x4 *>(base + 64 * k.hh + 16 * k.is);
        w.ql1 = *reinterpret_cast<const u32x4 *>(base + 64 * k.hh + 32 + 16 * k.is);
        w.qh = *reinterpret_cast<const u32x4 *>(base + 128 + 32 * k.hh + 16 * k.is);
        w.sc = *reinterpret_cast<const u32x2 *>(base + 192 + 8 * k.hh);
        w.sc2 = *reinterpret_cast<const uint32_t *>(base + 192 + 8 * k.hh + (off ? 8 : 4));  // aligned block: re-read
        w.d = ld2(blk + 208);
    }
    template <bool DUMP>
    static __device__ __forceinline__ float dot(const Wt &w, const Act &a, const Lane &k, int32_t *sums,
                                                uint32_t u, bool valid) {
        // sum (q - 32) a = sum q a - 32 sum a: the accumulators start at -32 sum a
        int p0 = a.nasum32[0], p1 = a.nasum32[1], p2 = a.nasum32[2], p3 = a.nasum32[3];
        // The dword after each of the lane's pieces.  The 16-byte pieces of a block in address order: ql 0..7
        // (lane (hh, is) holds 4hh + is in ql0 and 4hh + 2 + is in ql1), qh 8..11 (8 + 2hh + is), scales 12.
        // Lanes of a block are a quad: position 2hh + is.
        const uint32_t x_ql0 = qp<0xB1>(w.ql0[0]), x_ql1 = qp<0xB1>(w.ql1[0]), x_qh = qp<0xB1>(w.qh[0]);
        const uint32_t p2_ql0 = qp<0xAA>(w.ql0[0]), p2_qh = qp<0xAA>(w.qh[0]);  // quad position 2: (hh 1, is 0)
        const uint32_t p0_qh = qp<0x00>(w.qh[0]), p0_sc = qp<0x00>(w.sc[0]);     // quad position 0: (hh 0, is 0)
        const u32x4 ql0 = realign(w.ql0, k.is ? x_ql1 : x_ql0, w.sh);
        const u32x4 ql1 = realign(w.ql1, k.is ? (k.hh ? p0_qh : p2_ql0) : x_ql1, w.sh);
        const u32x4 qh = realign(w.qh, k.is ? (k.hh ? p0_sc : p2_qh) : x_qh, w.sh);
        for (int i = 0; i < 4; i++) {
            const uint32_t l0 = ql0[i], l1 = ql1[i], h = qh[i];
            // q6_k.rs:55-60, four bytes at a time.  hm holds the 2-bit fields of q1 (bits 0-1)
            // and q3 (bits 4-5) of every byte, hn those of q2 and q4; a bitfield insert under
            // the low-nibble mask joins them with the ql nibbles.
            const uint32_t hm = h & 0x33333333u, hn = (h >> 2) & 0x33333333u;
            const uint32_t q0 = (l0 & 0x0F0F0F0Fu) | ((hm << 4) & 0xF0F0F0F0u);
            const uint32_t q1 = (l1 & 0x0F0F0F0Fu) | ((hn << 4) & 0xF0F0F0F0u);
            const uint32_t q2 = ((l0 >> 4) & 0x0F0F0F0Fu) | (hm & 0xF0F0F0F0u);
            const uint32_t q3 = ((l1 >> 4) & 0x0F0F0F0Fu) | (hn & 0xF0F0F0F0u);
            p0 = sdot4(q0, a.q[0][i], p0);
            p1 = sdot4(q1, a.q[1][i], p1);
            p2 = sdot4(q2, a.q[2][i], p2);
            p3 = sdot4(q3, a.q[3][i], p3);
        }
        const int isum[4] = {p0, p1, p2, p3};
        // scales[8hh + is + 2j]: bytes is, is+2 of sc[0], then of sc[1]
        const uint32_t s0 = __builtin_amdgcn_alignbit(w.sc[1], w.sc[0], w.sh) >> (8 * k.is);
        const uint32_t s1 = __builtin_amdgcn_alignbit(w.sc2, w.sc[1], w.sh) >> (8 * k.is);
        const int scv[4] = {(int)(int8_t)(s0 & 0xFF), (int)(int8_t)((s0 >> 16) & 0xFF),
                            (int)(int8_t)(s1 & 0xFF), (int)(int8_t)((s1 >> 16) & 0xFF)};
        float t = 0.0f;
        for (int j = 0; j < 4; j++) {
            // |sc * isum| <= 128 * 16 * 63 * 128 < 2^24: exact as int24 operands and as fp32
            t = fmaf(a.d_a[j], (float)mul24(isum[j], scv[j]), t);
            if (DUMP && valid) sums[16 * (u >> 2) + 8 * k.hh + 2 * j + k.is] = isum[j];
        }
        return h2f(w.d) * t;
    }
};

// ---------------------------------------------------------------------------
// Q8_0 weights, Q/reference/q8_0.rs:36-41; fused form Q/simd/avx2/q8_0.rs:205,242.
// Unit = one 34-byte block against the activation block of the same index.
struct FmtQ8_0 {
    static constexpr uint32_t BLOCK_BYTES = 34, BLOCK_COLS = 32, UNIT_COLS = 32;
    static constexpr uint32_t TYPE_ID = OXQ_TYPE_Q8_0;
    static constexpr uint32_t TWO_ROW_BATCH_BYTES = 3400;  // two rows per batch up to this slice of a row per wave
    struct Lane {};
    struct Act {
        u32x4 q0, q1;
        float d_a;
    };
    // A block is 34 bytes, so every other one starts two bytes off a dword boundary.  Each lane issues
    // two dword-aligned 16-byte loads and one 2-byte load that together cover its 34 bytes exactly:
    //   block on a dword boundary: bytes 0..31 (d, payload 0..29) + the 2 bytes 32..33 (payload 30..31);
    //   block two bytes off:       bytes 2..33 (the payload, aligned as it is) + the 2 bytes 0..1 (d).
    // dot() shifts the first form into place (v_alignbit by 16; by 0 for the second form).
    struct Wt {
        u32x4 q0, q1;
        uint32_t x;    // the 2-byte load
        uint32_t off;  // 0: first form, else second
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
        w.off = (uint32_t)(reinterpret_cast<uintptr_t>(blk) & 2);  // blocks start on even addresses
        const uint8_t *base = blk + w.off;
        w.q0 = *reinterpret_cast<const u32x4 *>(base);
        w.q1 = *reinterpret_cast<const u32x4 *>(base + 16);
        w.x = ld2(w.off ? blk : blk + 32);
    }
    template <bool DUMP>
    static __device__ __forceinline__ float dot(const Wt &w, const Act &a, const Lane &, int32_t *sums,
                                                uint32_t u, bool valid) {
        const uint32_t sh = w.off ? 0u : 16u;
        const uint32_t dw[9] = {w.q0[0], w.q0[1], w.q0[2], w.q0[3], w.q1[0], w.q1[1], w.q1[2], w.q1[3], w.x};
        int p = 0;
        for (int i = 0; i < 4; i++) {
            p = sdot4(__builtin_amdgcn_alignbit(dw[i + 1], dw[i], sh), a.q0[i], p);
            p = sdot4(__builtin_amdgcn_alignbit(dw[i + 5], dw[i + 4], sh), a.q1[i], p);
        }
        if (DUMP && valid) sums[u] = p;
        const uint32_t dbits = w.off ? w.x : (w.q0[0] & 0xFFFFu);
        const float scale = h2f(dbits) * a.d_a;  // avx2/q8_0.rs:205
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
    static constexpr uint32_t TYPE_ID = OXQ_TYPE_Q4_0;
    static constexpr uint32_t TWO_ROW_BATCH_BYTES = 3400;  // two rows per batch up to this slice of a row per wave
    struct Lane {};
    struct Act {
        uint32_t ev[4], od[4];
        float d_a;
        int nasum8;  // -8 * sum of the 32 activation bytes
    };
    // 18-byte blocks, loaded as FmtQ8_0 loads its 34: one dword-aligned 16-byte load (bytes 0..15 of a
    // block on a dword boundary, bytes 2..17 of one two bytes off) and one 2-byte load for the rest.
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
        int s = 0;
        for (int i = 0; i < 4; i++) {
            s = sdot4(q0[i], 0x01010101u, s);
            s = sdot4(q1[i], 0x01010101u, s);
        }
        a.nasum8 = -8 * s;
        a.d_a = valid ? h2f(dbits) : 0.0f;
    }
    static __device__ __forceinline__ void load_w(Wt &w, const uint8_t *row, uint32_t u, const Lane &) {
        const uint8_t *blk = row + (size_t)u * BLOCK_BYTES;
        w.off = (uint32_t)(reinterpret_cast<uintptr_t>(blk) & 2);
        w.q = *reinterpret_cast<const u32x4 *>(blk + w.off);
        w.x = ld2(w.off ? blk : blk + 16);
    }
    template <bool DUMP>
    static __device__ __forceinline__ float dot(const Wt &w, const Act &a, const Lane &, int32_t *sums,
                                                uint32_t u, bool valid) {
        const uint32_t sh = w.off ? 0u : 16u;
        const uint32_t dw[5] = {w.q[0], w.q[1], w.q[2], w.q[3], w.x};
        int p = a.nasum8;
        for (int i = 0; i < 4; i++) {
            const uint32_t q = __builtin_amdgcn_alignbit(dw[i + 1], dw[i], sh);
            p = sdot4(q & 0x0F0F0F0Fu, a.ev[i], p);
            p = sdot4((q >> 4) & 0x0F0F0F0Fu, a.od[i], p);
        }
        if (DUMP && valid) sums[u] = p;
        const float scale = h2f(w.off ? w.x : (w.q[0] & 0xFFFFu)) * a.d_a;  // avx2/q4_0.rs:211
        return scale * (float)p;               // avx2/q4_0.rs:265
    }
};

// ---------------------------------------------------------------------------
// IQ4_XS, Q/reference/iq4_xs.rs:47-97; codebook Q/reference/iq_shared.rs:16-18.
// 136 B = f16 d, u16 scales_h, 4 B scales_l, 128 B nibble indices.  Unit = one
// 32-weight sub-block i: qs[16i..16i+16], interleaved nibbles.  Term:
// d * float((ls - 32) * sum kvalues[idx] * a) * d_a.
struct FmtIQ4XS {
    static constexpr uint32_t BLOCK_BYTES = 136, BLOCK_COLS = 256, UNIT_COLS = 32;
    static constexpr uint32_t TYPE_ID = OXQ_TYPE_IQ4_XS;
    static constexpr uint32_t TWO_ROW_BATCH_BYTES = 3400;  // two rows per batch up to this slice of a row per wave
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
    template <class SRC>
    static __device__ __forceinline__ void load_act(Act &a, const SRC &src, uint32_t u, bool valid, const Lane &) {
        u32x4 q0, q1;
        uint32_t dbits;
        src.block(u, q0, q1, dbits);
        split_even_odd(q0, q1, a.ev, a.od);
        a.d_a = valid ? h2f(dbits) : 0.0f;
    }
    static __device__ __forceinline__ void load_w(Wt &w, const uint8_t *row, uint32_t u, const Lane &k) {
        const uint8_t *blk = row + (size_t)(u >> 3) * BLOCK_BYTES;
        w.hdr = ld8(blk);
        w.q = ld16(blk + 8 + 16 * k.i);
    }
    // Four 4-bit indices (one per byte) -> four codebook bytes: two 8-entry byte
    // permutes, then a third permute picks the upper table where bit 3 is set.
    static __device__ __forceinline__ uint32_t lut4(uint32_t idx) {
        const uint32_t T0 = 0xBFAD9881u, T1 = 0xF6EADDCFu, T2 = 0x26190D01u, T3 = 0x71594535u;
        const uint32_t sel = idx & 0x07070707u;
        const uint32_t lo = __builtin_amdgcn_perm(T1, T0, sel);
        const uint32_t hi = __builtin_amdgcn_perm(T3, T2, sel);
        // the identity selector in a vector register: (x >> 1 & mask) | base is then one v_and_or_b32 (an
        // instruction takes a single scalar operand, and both constants would be scalars otherwise)
        uint32_t base;
        asm("v_mov_b32 %0, 0x03020100" : "=v"(base));
        return __builtin_amdgcn_perm(hi, lo, ((idx >> 1) & 0x04040404u) | base);
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
        // |ls * p| <= 32 * 32 * 127 * 128 < 2^24: exact
        return h2f(w.hdr[0] & 0xFFFF) * ((float)mul24(p, ls) * a.d_a);
    }
};

}  // namespace oxq
