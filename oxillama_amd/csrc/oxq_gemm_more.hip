// The int8-MFMA tile kernel (oxq_gemm_tile.hpp) instantiated for further formats: Q5_K, Q4_1, Q5_0,
// Q5_1, Q8_1, IQ4_NL, Q3_K, Q2_K, and the few-token kernel (oxq_gemm_skinny.hpp) for all of them
// but Q8_1.  Each is a small policy (which bytes a lane fetches per group of two
// sub-blocks, how they become int8 B operands, how the scale factors are decoded, which byte
// order the activations need); kernel body, tile shapes and launch policy are shared.  A
// translation unit of its own so that the two sets compile side by side; only the default tile
// shapes are instantiated here.
#define OXQ_TILE_DEFAULT_SHAPES_ONLY
#include "oxq_formats_more.hpp"
#include "oxq_gemm_skinny.hpp"

namespace oxq {

// Q5_K (reference/q5_k.rs:27-102): 176 B = d, dmin, 12 B of 6-bit scales/mins, 32 B qh, 128 B
// nibbles.  As Q4_K: the lane's 16 bytes qs[32g + 16h ..] carry weights 16h..16h+15 of sub-block 2g
// (low nibbles) and 2g+1 (high); their fifth bits are bits g and g+4 of qh[16h ..].
struct TileQ5K {
    static constexpr uint32_t TYPE = OXQ_TYPE_Q5_K, BLOCK_BYTES = 176;
    static constexpr bool HAS_MIN = true;
    static constexpr int ACT_PERM = 0, NQ = 2, KSPLIT = 1;
    using Hdr = TileQ4K::Hdr;
    static __device__ __forceinline__ uint32_t sub_block(uint32_t g, uint32_t e) { return 2 * g + e; }
    static __device__ __forceinline__ void fetch(__amdgpu_buffer_rsrc_t rs, uint32_t row_off, uint32_t h, uint32_t so_blk,
                                                 uint32_t g, u32x4 (&qs)[NQ]) {
        qs[0] = buf16(rs, row_off + 16 * h, so_blk + 48 + 32 * g);
        qs[1] = buf16(rs, row_off + 16 * h, so_blk + 16);
    }
    template <int SPL>
    static __device__ __forceinline__ void load_hdr(__amdgpu_buffer_rsrc_t rs, uint32_t row_off, uint32_t so_blk, uint32_t s0,
                                                    Hdr &hd) {
        TileQ4K::load_hdr<SPL>(rs, row_off, so_blk, s0, hd);
    }
    static __device__ __forceinline__ void factors(const Hdr &hd, uint32_t e, uint32_t s, float (&dsc)[KSPLIT], float &qneg) {
        TileQ4K::factors(hd, e, s, dsc, qneg);  // same header layout (reference/q5_k.rs:27-49)
    }
    static __device__ __forceinline__ void operands(const u32x4 (&qs)[NQ], uint32_t g, BOperand<1> (&bop)[2]) {
        for (int i = 0; i < 4; i++) {
            const uint32_t hb = qs[1][i] >> g;
            bop[0].k32[i] = (int)((qs[0][i] & 0x0F0F0F0Fu) | ((hb & 0x01010101u) << 4));
            bop[1].k32[i] = (int)(((qs[0][i] >> 4) & 0x0F0F0F0Fu) | (hb & 0x10101010u));
        }
    }
};

// The few-token kernel's view of the same block (oxq_gemm_skinny.hpp): lane (c, q) takes bytes 8q..8q+7 of each run of
// 32 nibble bytes and of qh (the fifth bits of weights 8q..8q+7 of every sub-block: bits g and g + 4 of byte l belong to
// weight l of sub-blocks 2g and 2g + 1).  352 bytes of a row per step leave LDS for one token tile at two work groups per compute unit.
template <>
struct Skinny<TileQ5K> {
    static constexpr bool OK = true;
    static constexpr uint32_t BLOCK = 176, ROW_STRIDE = 368;
    static constexpr bool HAS_MIN = true, TABLE = true, ONE_TILE = true;
    static constexpr int ACT_PERM = 0, KSPLIT = 1;
    struct Raw {
        u32x4 hdr;
        u32x2 qh;
        u32x2 qs[4];
    };
    static __device__ __forceinline__ void read_hdr(Raw &w, const uint8_t *blk, uint32_t) {
        w.hdr = *reinterpret_cast<const u32x4 *>(blk);
    }
    template <int U>
    static __device__ __forceinline__ void read(Raw &w, const uint8_t *blk, uint32_t q) {
        w.qh = *reinterpret_cast<const u32x2 *>(blk + 16 + 8 * q);
#pragma unroll
        for (int g = 0; g < 4; g++) w.qs[g] = *reinterpret_cast<const u32x2 *>(blk + 48 + 32 * g + 8 * q);
    }
    static __device__ __forceinline__ long operand(const Raw &w, int s) {
        const u32x2 v = w.qs[s >> 1];
        const int bit = (s >> 1) + 4 * (s & 1);  // (reference/q5_k.rs:86,93: bit g for the low nibbles of run g, g + 4 for the high)
        const uint32_t lo = ((s & 1) ? (v[0] >> 4) & 0x0F0F0F0Fu : v[0] & 0x0F0F0F0Fu) | (((w.qh[0] >> bit) & 0x01010101u) << 4);
        const uint32_t hi = ((s & 1) ? (v[1] >> 4) & 0x0F0F0F0Fu : v[1] & 0x0F0F0F0Fu) | (((w.qh[1] >> bit) & 0x01010101u) << 4);
        return (long)(((uint64_t)hi << 32) | lo);
    }
    static __device__ __forceinline__ void factors(const Raw &w, uint32_t half, int i, float &dsc, float &qneg) {
        TileQ4K::Hdr hd;
        hd.w = w.hdr;
        float d1[1];
        TileQ4K::factors(hd, 0, 4 * half + i, d1, qneg);  // (the header of Q4_K)
        dsc = d1[0];
    }
};

// 32-weight blocks of interleaved nibbles (byte j = weights 2j, 2j+1), eight blocks per 256-weight
// step: Q4_1 (reference/q4_1.rs:37-46: 20 B = d, m, 16 B; w = d * q + m, the "+ m" through the
// zero-point term) and IQ4_NL (reference/iq4_nl.rs:43-51: 18 B = d, 16 B of codebook indices).
template <uint32_t TYPE_ID, uint32_t STRIDE, uint32_t PAYLOAD, bool LUT, bool WITH_M>
struct TileNibbles32 {
    static constexpr uint32_t TYPE = TYPE_ID, BLOCK_BYTES = 8 * STRIDE;
    static constexpr bool RAGGED_K = true;
    static constexpr bool HAS_MIN = WITH_M;
    static constexpr int ACT_PERM = 1, NQ = 1, KSPLIT = 1;
    struct Hdr {
        uint32_t d[8], m[8];  // f16 bits of the lane's sub-blocks
    };
    static __device__ __forceinline__ uint32_t sub_block(uint32_t g, uint32_t e) { return 2 * g + e; }
    static __device__ __forceinline__ void fetch(__amdgpu_buffer_rsrc_t rs, uint32_t row_off, uint32_t h, uint32_t so_blk,
                                                 uint32_t g, u32x4 (&qs)[NQ]) {
        if constexpr ((STRIDE + 2) % 4 == 0 && PAYLOAD % 4 == 2)  // half 0 starts 2 past a dword boundary, half 1 on one
            qs[0] = buf16_shift(rs, row_off + (STRIDE + 2) * h, so_blk + 2 * STRIDE * g + PAYLOAD - 2, h ? 0u : 16u);
        else
            qs[0] = buf16(rs, row_off + STRIDE * h, so_blk + 2 * STRIDE * g + PAYLOAD);  // block 2g + h
    }
    template <int SPL>
    static __device__ __forceinline__ void load_hdr(__amdgpu_buffer_rsrc_t rs, uint32_t row_off, uint32_t so_blk, uint32_t s0,
                                                    Hdr &hd) {
#pragma unroll
        for (int e = 0; e < SPL; e++) {
            hd.d[e] = (uint32_t)(uint16_t)__builtin_amdgcn_raw_buffer_load_b16(rs, row_off + STRIDE * (s0 + e), so_blk, 0);
            if (WITH_M)
                hd.m[e] = (uint32_t)(uint16_t)__builtin_amdgcn_raw_buffer_load_b16(rs, row_off + STRIDE * (s0 + e) + 2, so_blk, 0);
        }
    }
    static __device__ __forceinline__ void factors(const Hdr &hd, uint32_t e, uint32_t, float (&dsc)[KSPLIT], float &qneg) {
        dsc[0] = h2f(hd.d[e]);
        qneg = WITH_M ? h2f(hd.m[e]) : 0.0f;
    }
    static __device__ __forceinline__ void operands(const u32x4 (&qs)[NQ], uint32_t, BOperand<1> (&bop)[2]) {
        uint32_t x[2][2];
        halves_to_pieces(qs[0], x);
        for (int e = 0; e < 2; e++)
            for (int i = 0; i < 2; i++) {
                const uint32_t lo = x[e][i] & 0x0F0F0F0Fu, hi = (x[e][i] >> 4) & 0x0F0F0F0Fu;
                bop[e].k32[2 * i] = (int)(LUT ? FmtIQ4XS::lut4(lo) : lo);
                bop[e].k32[2 * i + 1] = (int)(LUT ? FmtIQ4XS::lut4(hi) : hi);
            }
    }
};
using TileQ4_1 = TileNibbles32<OXQ_TYPE_Q4_1, 20, 4, false, true>;
using TileIQ4NL = TileNibbles32<OXQ_TYPE_IQ4_NL, 18, 2, true, false>;

// Q8_1 (reference/q8_1.rs:36-42): 36 B = d, s (unused), 32 int8; the payload is the B operand.
struct TileQ8_1 {
    static constexpr uint32_t TYPE = OXQ_TYPE_Q8_1, BLOCK_BYTES = 8 * 36;
    static constexpr bool RAGGED_K = true;
    static constexpr bool HAS_MIN = false;
    static constexpr int ACT_PERM = 0, NQ = 2, KSPLIT = 1;
    using Hdr = TileQ8_0::Hdr;
    static __device__ __forceinline__ uint32_t sub_block(uint32_t g, uint32_t e) { return 2 * g + e; }
    static __device__ __forceinline__ void fetch(__amdgpu_buffer_rsrc_t rs, uint32_t row_off, uint32_t h, uint32_t so_blk,
                                                 uint32_t g, u32x4 (&qs)[NQ]) {
        qs[0] = buf16(rs, row_off + 16 * h, so_blk + 72 * g + 4);
        qs[1] = buf16(rs, row_off + 16 * h, so_blk + 72 * g + 40);
    }
    template <int SPL>
    static __device__ __forceinline__ void load_hdr(__amdgpu_buffer_rsrc_t rs, uint32_t row_off, uint32_t so_blk, uint32_t s0,
                                                    Hdr &hd) {
#pragma unroll
        for (int e = 0; e < SPL; e++)
            hd.d[e] = (uint32_t)(uint16_t)__builtin_amdgcn_raw_buffer_load_b16(rs, row_off + 36 * (s0 + e), so_blk, 0);
    }
    static __device__ __forceinline__ void factors(const Hdr &hd, uint32_t e, uint32_t, float (&dsc)[KSPLIT], float &qneg) {
        dsc[0] = h2f(hd.d[e]);
        qneg = 0.0f;
    }
    static __device__ __forceinline__ void operands(const u32x4 (&qs)[NQ], uint32_t, BOperand<1> (&bop)[2]) {
        for (int e = 0; e < 2; e++)
            for (int i = 0; i < 4; i++) bop[e].k32[i] = (int)qs[e][i];
    }
};

// Q5_0 / Q5_1 (reference/q5_0.rs:39-55, q5_1.rs:38-56): d [, m], u32 qh, 16 B of nibbles; byte j holds
// the low four bits of weights j (low nibble) and j + 16 (high nibble), bit j / j + 16 of qh the
// fifth.  Lane half h fetches block 2g + h whole; after the exchange every lane holds bytes
// 8h..8h+7 of both blocks, i.e. weights {8h..8h+7, 16+8h..23+8h}: the k-slot order the preparation
// kernel stores under ACT_PERM = 2.  Q5_0's "- 16" and Q5_1's "+ m" go through the zero-point term.
template <uint32_t TYPE_ID, uint32_t STRIDE, bool WITH_M>
struct TileQ5x {
    static constexpr uint32_t TYPE = TYPE_ID, BLOCK_BYTES = 8 * STRIDE;
    static constexpr bool RAGGED_K = true;
    static constexpr uint32_t QH = WITH_M ? 4 : 2, PAYLOAD = QH + 4;
    static constexpr bool HAS_MIN = true;
    static constexpr int ACT_PERM = 2, NQ = 2, KSPLIT = 1;
    using Hdr = typename TileNibbles32<TYPE_ID, STRIDE, PAYLOAD, false, WITH_M>::Hdr;
    static __device__ __forceinline__ uint32_t sub_block(uint32_t g, uint32_t e) { return 2 * g + e; }
    static __device__ __forceinline__ void fetch(__amdgpu_buffer_rsrc_t rs, uint32_t row_off, uint32_t h, uint32_t so_blk,
                                                 uint32_t g, u32x4 (&qs)[NQ]) {
        if constexpr ((STRIDE + 2) % 4 == 0 && PAYLOAD % 4 == 2)  // Q5_0: half 0 starts 2 past a dword boundary, half 1 on one
            qs[0] = buf16_shift(rs, row_off + (STRIDE + 2) * h, so_blk + 2 * STRIDE * g + PAYLOAD - 2, h ? 0u : 16u);
        else
            qs[0] = buf16(rs, row_off + STRIDE * h, so_blk + 2 * STRIDE * g + PAYLOAD);  // block 2g + h: nibbles
        qs[1] = u32x4{(uint32_t)__builtin_amdgcn_raw_buffer_load_b32(rs, row_off + STRIDE * h, so_blk + 2 * STRIDE * g + QH, 0),
                      0, 0, 0};                                                          // and its qh
    }
    template <int SPL>
    static __device__ __forceinline__ void load_hdr(__amdgpu_buffer_rsrc_t rs, uint32_t row_off, uint32_t so_blk, uint32_t s0,
                                                    Hdr &hd) {
        TileNibbles32<TYPE_ID, STRIDE, PAYLOAD, false, WITH_M>::template load_hdr<SPL>(rs, row_off, so_blk, s0, hd);
    }
    static __device__ __forceinline__ void factors(const Hdr &hd, uint32_t e, uint32_t, float (&dsc)[KSPLIT], float &qneg) {
        dsc[0] = h2f(hd.d[e]);
        qneg = WITH_M ? h2f(hd.m[e]) : -(16.0f * dsc[0]);  // exact
    }
    static __device__ __forceinline__ void operands(const u32x4 (&qs)[NQ], uint32_t, BOperand<1> (&bop)[2]) {
        uint32_t x[2][2];
        halves_to_pieces(qs[0], x);
        // qh of block 2g in every lane (s[0]) and of block 2g + 1 (s[1])
        const auto s = __builtin_amdgcn_permlane32_swap(qs[1][0], qs[1][0], false, false);
        const uint32_t hsel = (__lane_id() >> 5) * 8;  // this half's byte of the low / high 16 fifth bits
        for (int e = 0; e < 2; e++) {
            const uint32_t lo8 = ((uint32_t)s[e] >> hsel) & 0xFFu, hi8 = ((uint32_t)s[e] >> (16 + hsel)) & 0xFFu;
            bop[e].k32[0] = (int)((x[e][0] & 0x0F0F0F0Fu) | (spread4(lo8 & 0xFu) << 4));
            bop[e].k32[1] = (int)((x[e][1] & 0x0F0F0F0Fu) | (spread4(lo8 >> 4) << 4));
            bop[e].k32[2] = (int)(((x[e][0] >> 4) & 0x0F0F0F0Fu) | (spread4(hi8 & 0xFu) << 4));
            bop[e].k32[3] = (int)(((x[e][1] >> 4) & 0x0F0F0F0Fu) | (spread4(hi8 >> 4) << 4));
        }
    }
};
using TileQ5_0 = TileQ5x<OXQ_TYPE_Q5_0, 22, false>;
using TileQ5_1 = TileQ5x<OXQ_TYPE_Q5_1, 24, true>;

// Q3_K (reference/q3_k.rs:30-109): 110 B = 32 B hmask, 64 B of 2-bit fields, 12 B of 6-bit scales
// (one per 16 weights, minus 32), d.  Sub-block s = 4n + j (32 weights) takes bits 2j..2j+1 of
// qs[32n + l] and bit s of hmask[l], l = 0..31; weight = (q2 | hbit << 2) - 4.  As Q6_K: lane (c, h)
// fetches bytes 16h..16h+15 (the 16-weight half h, which has its own scale), halves_to_pieces
// hands every lane bytes 8h..8h+7 of both halves -- the k-slot order of the K = 16 operands and
// of the activations (ACT_PERM = 2).  Group g = sub-blocks 2g and 2g+1 (n = g / 2).
struct TileQ3K {
    static constexpr uint32_t TYPE = OXQ_TYPE_Q3_K, BLOCK_BYTES = 110;
    static constexpr bool HAS_MIN = false;
    static constexpr int ACT_PERM = 2, NQ = 2, KSPLIT = 2;
    struct Hdr {
        uint32_t s[3];  // the 12 scale bytes
        uint32_t d;     // f16 bits
    };
    static __device__ __forceinline__ uint32_t sub_block(uint32_t g, uint32_t e) { return 2 * g + e; }
    static __device__ __forceinline__ void fetch(__amdgpu_buffer_rsrc_t rs, uint32_t row_off, uint32_t h, uint32_t so_blk,
                                                 uint32_t g, u32x4 (&qs)[NQ]) {
        qs[0] = buf16(rs, row_off + 16 * h, so_blk + 32 + 32 * (g >> 1));
        qs[1] = buf16(rs, row_off + 16 * h, so_blk);
    }
    template <int SPL>
    static __device__ __forceinline__ void load_hdr(__amdgpu_buffer_rsrc_t rs, uint32_t row_off, uint32_t so_blk, uint32_t,
                                                    Hdr &hd) {
        for (int i = 0; i < 3; i++) hd.s[i] = (uint32_t)__builtin_amdgcn_raw_buffer_load_b32(rs, row_off, so_blk + 96 + 4 * i, 0);
        hd.d = (uint32_t)(uint16_t)__builtin_amdgcn_raw_buffer_load_b16(rs, row_off, so_blk + 108, 0);
    }
    // decode_scales (reference/q3_k.rs:30-59) for index 2s + is = 8n + kk: n = 0: s[kk] & 63;
    // n = 1: nibble (kk >> 2) of s[8 + (kk & 3)] | (s[kk] >> 6) << 4; each minus 32.
    static __device__ __forceinline__ void factors(const Hdr &hd, uint32_t, uint32_t s, float (&dsc)[KSPLIT], float &qneg) {
        const float d = h2f(hd.d);
        for (int is = 0; is < 2; is++) {
            const uint32_t idx = 2 * s + is, kk = idx & 7;
            const uint32_t byte = ((kk < 4 ? hd.s[0] : hd.s[1]) >> (8 * (kk & 3))) & 0xFF;
            const uint32_t hi = ((hd.s[2] >> (8 * (kk & 3) + 4 * (kk >> 2))) & 0x0F) | ((byte >> 6) << 4);
            dsc[is] = d * (float)((int)(idx < 8 ? (byte & 0x3F) : hi) - 32);  // exact
        }
        qneg = 0.0f;
    }
    static __device__ __forceinline__ void operands(const u32x4 (&qs)[NQ], uint32_t g, BOperand<2> (&bop)[2]) {
        uint32_t l[2][2], hb[2][2];
        halves_to_pieces(qs[0], l);
        halves_to_pieces(qs[1], hb);
        for (int e = 0; e < 2; e++) {
            const uint32_t j = 2 * (g & 1) + e, s = 2 * g + e;
            for (int is = 0; is < 2; is++) {
                uint32_t q[2];
                for (int i = 0; i < 2; i++) {
                    const uint32_t v = ((l[is][i] >> (2 * j)) & 0x03030303u) | (((hb[is][i] >> s) & 0x01010101u) << 2);
                    // v - 4 per byte (0..7 -> -4..3) without carries between bytes
                    q[i] = ((v | 0x80808080u) - 0x04040404u) ^ 0x80808080u;
                }
                bop[e].k16[is] = (long)(((uint64_t)q[1] << 32) | q[0]);
            }
        }
    }
};

// Q2_K (reference/q2_k.rs:31-105): 84 B = 16 scale bytes (low nibble: scale, high nibble: min, one
// per 16 weights), 64 B of 2-bit fields, d, dmin.  Same walk as Q3_K without the high bit; weight =
// d * sc * q2 - dmin * mn, the second part through the zero-point term with one factor per
// 16-weight half (MIN_PLANES = 2).
struct TileQ2K {
    static constexpr uint32_t TYPE = OXQ_TYPE_Q2_K, BLOCK_BYTES = 84;
    static constexpr bool HAS_MIN = true;
    static constexpr int ACT_PERM = 2, NQ = 1, KSPLIT = 2, MIN_PLANES = 2;
    struct Hdr {
        u32x4 sc;     // the 16 scale bytes
        uint32_t dd;  // d | dmin << 16 (f16 bits)
    };
    static __device__ __forceinline__ uint32_t sub_block(uint32_t g, uint32_t e) { return 2 * g + e; }
    static __device__ __forceinline__ void fetch(__amdgpu_buffer_rsrc_t rs, uint32_t row_off, uint32_t h, uint32_t so_blk,
                                                 uint32_t g, u32x4 (&qs)[NQ]) {
        qs[0] = buf16(rs, row_off + 16 * h, so_blk + 16 + 32 * (g >> 1));
    }
    template <int SPL>
    static __device__ __forceinline__ void load_hdr(__amdgpu_buffer_rsrc_t rs, uint32_t row_off, uint32_t so_blk, uint32_t,
                                                    Hdr &hd) {
        hd.sc = buf16(rs, row_off, so_blk);
        hd.dd = (uint32_t)__builtin_amdgcn_raw_buffer_load_b32(rs, row_off, so_blk + 80, 0);
    }
    // scales[2s + is]: low nibble the scale, high nibble the min (reference/q2_k.rs:60-75)
    static __device__ __forceinline__ void factors2(const Hdr &hd, uint32_t, uint32_t s, float (&dsc)[KSPLIT],
                                                    float (&qneg)[2]) {
        const uint32_t pair = hd.sc[s >> 1] >> (16 * (s & 1));
        const float d = h2f(hd.dd & 0xFFFF), dmin = h2f(hd.dd >> 16);
        for (int is = 0; is < 2; is++) {
            const uint32_t byte = (pair >> (8 * is)) & 0xFF;
            dsc[is] = d * (float)(byte & 0x0F);        // exact
            qneg[is] = -(dmin * (float)(byte >> 4));   // exact
        }
    }
    static __device__ __forceinline__ void operands(const u32x4 (&qs)[NQ], uint32_t g, BOperand<2> (&bop)[2]) {
        uint32_t l[2][2];
        halves_to_pieces(qs[0], l);
        for (int e = 0; e < 2; e++) {
            const uint32_t j = 2 * (g & 1) + e;
            for (int is = 0; is < 2; is++) {
                const uint32_t q0 = (l[is][0] >> (2 * j)) & 0x03030303u, q1 = (l[is][1] >> (2 * j)) & 0x03030303u;
                bop[e].k16[is] = (long)(((uint64_t)q1 << 32) | q0);
            }
        }
    }
};

int tile_act_perm_more(uint32_t type) {
    switch (type) {
    case OXQ_TYPE_Q4_1:
    case OXQ_TYPE_IQ4_NL: return 1;
    case OXQ_TYPE_Q5_0:
    case OXQ_TYPE_Q5_1:
    case OXQ_TYPE_Q3_K:
    case OXQ_TYPE_Q2_K: return 2;
    default: return 0;
    }
}

bool tile_needs_p16_more(uint32_t type) { return type == OXQ_TYPE_Q2_K; }

// Q3_K in the few-token kernel, as Q6_K there (two scale factors per 32-weight sub-block, one MFMA per 16-weight half,
// the operand unsigned -- 0..7 -- and the "- 4" in the MFMA's addend).  Lane (c, q) takes weights 8q..8q+7 of every
// sub-block: bytes 8q..8q+7 of hmask (bit s = sub-block s) and of each run of 32 bytes of 2-bit fields (run n,
// bits 2j..2j+1 = sub-block 4n + j).  The step's second block starts 110 bytes into the row's strip, 6 past a multiple
// of 8.  272 bytes = 68 dwords per row: the 64 lanes of an 8-byte read hit different banks.
template <>
struct Skinny<TileQ3K> {
    static constexpr bool OK = true;
    static constexpr uint32_t BLOCK = 110, ROW_STRIDE = 272;
    static constexpr bool HAS_MIN = false, TABLE = true, ONE_TILE = true;
    static constexpr int ACT_PERM = 0, KSPLIT = 2, OFFSET = 4;
    struct Raw {
        u32x2 hm, qs[2];
    };
    template <int U>
    static __device__ __forceinline__ void read(Raw &w, const uint8_t *blk, uint32_t q) {
        w.hm = strip_get8<6 * U>(blk + 8 * q);
#pragma unroll
        for (int n = 0; n < 2; n++) w.qs[n] = strip_get8<6 * U>(blk + 32 + 32 * n + 8 * q);
    }
    static __device__ __forceinline__ long operand(const Raw &w, int s) {
        const u32x2 l = w.qs[s >> 2];
        uint32_t v[2];
#pragma unroll
        for (int i = 0; i < 2; i++)
            v[i] = ((l[i] >> (2 * (s & 3))) & 0x03030303u) | (((w.hm[i] >> s) & 0x01010101u) << 2);
        return (long)(((uint64_t)v[1] << 32) | v[0]);
    }
    // Lane (c, q) decodes row c's scales 4q .. 4q + 3 (scale 2s + half belongs to that half of sub-block s):
    // decode_scales, reference/q3_k.rs:30-59 -- index 8n + kk: n = 0 the low six bits of byte kk; n = 1 nibble kk / 4 of
    // byte 8 + kk % 4, with the top two bits of byte kk above it; each minus 32.
    template <int U>
    static __device__ __forceinline__ void block_factors(const uint8_t *blk, uint32_t q, float (&f)[4]) {
        const uint32_t sw = strip_get4<2 * U>(blk + 96 + 4 * (q & 1)), s2 = strip_get4<2 * U>(blk + 104);
        const float d = h2f(reinterpret_cast<const StripR2 *>(blk + 108)->v);
#pragma unroll
        for (int b = 0; b < 4; b++) {
            const uint32_t byte = (sw >> (8 * b)) & 0xFF;
            const uint32_t hi = ((s2 >> (8 * b + 4 * (q & 1))) & 0x0F) | ((byte >> 6) << 4);
            f[b] = d * (float)((int)(q < 2 ? (byte & 0x3F) : hi) - 32);  // exact
        }
    }
};

// Q2_K in the few-token kernel: the walk of Q3_K without the high bit (lane (c, q): bytes 8q..8q+7 of each run of 32
// bytes of 2-bit fields; the second block of a step starts 84 bytes into the strip row, 4 past a multiple of 8), the
// operand the field itself, and per 16 weights a scale and a zero-point factor: the latter through a 16 x 16 x 4 fp32
// MFMA per four halves against P of the tokens' halves.  176 bytes = 44 dwords per strip row.
template <>
struct Skinny<TileQ2K> {
    static constexpr bool OK = true;
    static constexpr uint32_t BLOCK = 84, ROW_STRIDE = 176;
    static constexpr bool HAS_MIN = true, TABLE = true, ONE_TILE = true;
    static constexpr int ACT_PERM = 0, KSPLIT = 2, OFFSET = 0;
    struct Raw {
        u32x2 qs[2];
    };
    template <int U>
    static __device__ __forceinline__ void read(Raw &w, const uint8_t *blk, uint32_t q) {
#pragma unroll
        for (int n = 0; n < 2; n++) w.qs[n] = strip_get8<4 * U>(blk + 16 + 32 * n + 8 * q);
    }
    static __device__ __forceinline__ long operand(const Raw &w, int s) {
        const u32x2 l = w.qs[s >> 2];
        const uint32_t lo = (l[0] >> (2 * (s & 3))) & 0x03030303u, hi = (l[1] >> (2 * (s & 3))) & 0x03030303u;
        return (long)(((uint64_t)hi << 32) | lo);
    }
    // Lane (c, q): row c's scale bytes 4q .. 4q + 3 (byte 2s + half: low nibble the scale, high nibble the min of that
    // half of sub-block s; reference/q2_k.rs:60-75)
    template <int U>
    static __device__ __forceinline__ void block_factors(const uint8_t *blk, uint32_t q, float (&f)[4], float (&mn)[4]) {
        const uint32_t sc = *reinterpret_cast<const uint32_t *>(blk + 4 * q);
        const uint32_t dd = *reinterpret_cast<const uint32_t *>(blk + 80);
        const float d = h2f(dd & 0xFFFF), dmin = h2f(dd >> 16);
#pragma unroll
        for (int b = 0; b < 4; b++) {
            const uint32_t byte = (sc >> (8 * b)) & 0xFF;
            f[b] = d * (float)(byte & 0x0F);        // exact
            mn[b] = -(dmin * (float)(byte >> 4));   // exact
        }
    }
};

// Q4_1 and IQ4_NL in the few-token kernel, as Q4_0 there: lane (c, q) takes bytes 4q..4q+3 of each block's nibbles
// (weights 8q + {0,2,4,6} from the low nibbles, 8q + {1,3,5,7} from the high ones: the tokens' bytes even, then odd).
// Q4_1 (20-byte blocks, every field on a dword boundary): the "+ m" through the zero-point term.  336 bytes = 84
// dwords per strip row: the 64 lanes of a dword read hit different banks.
template <>
struct Skinny<TileQ4_1> {
    static constexpr bool OK = true;
    static constexpr uint32_t BLOCK = 160, ROW_STRIDE = 336;
    static constexpr bool HAS_MIN = true, TABLE = true, ONE_TILE = false;
    static constexpr int ACT_PERM = 1, KSPLIT = 1;
    struct Raw {
        uint32_t dm[4];  // d | m << 16 (f16 bits)
        uint32_t qs[8];
    };
    static __device__ __forceinline__ void read_hdr(Raw &w, const uint8_t *blk, uint32_t half) {
#pragma unroll
        for (int i = 0; i < 4; i++) w.dm[i] = *reinterpret_cast<const uint32_t *>(blk + 20 * (4 * half + i));
    }
    static __device__ __forceinline__ void factors(const Raw &w, uint32_t, int i, float &dsc, float &qneg) {
        dsc = h2f(w.dm[i] & 0xFFFF);
        qneg = h2f(w.dm[i] >> 16);
    }
    template <int U>
    static __device__ __forceinline__ void read(Raw &w, const uint8_t *blk, uint32_t q) {
#pragma unroll
        for (int s = 0; s < 8; s++) w.qs[s] = *reinterpret_cast<const uint32_t *>(blk + 20 * s + 4 + 4 * q);
    }
    static __device__ __forceinline__ long operand(const Raw &w, int s) {
        const uint32_t lo = w.qs[s] & 0x0F0F0F0Fu, hi = (w.qs[s] >> 4) & 0x0F0F0F0Fu;
        return (long)(((uint64_t)hi << 32) | lo);
    }
};
// IQ4_NL (18-byte blocks, the nibbles 2 past a dword boundary in the even blocks): the codebook byte is the operand.
template <>
struct Skinny<TileIQ4NL> {
    static constexpr bool OK = true;
    static constexpr uint32_t BLOCK = 144, ROW_STRIDE = 304;
    static constexpr bool HAS_MIN = false, TABLE = true, ONE_TILE = false;
    static constexpr int ACT_PERM = 1, KSPLIT = 1;
    struct Raw {
        uint32_t d[4];
        uint32_t qs[8];
    };
    static __device__ __forceinline__ void read_hdr(Raw &w, const uint8_t *blk, uint32_t half) {
#pragma unroll
        for (int i = 0; i < 4; i++) w.d[i] = reinterpret_cast<const StripR2 *>(blk + 18 * (4 * half + i))->v;
    }
    static __device__ __forceinline__ void factors(const Raw &w, uint32_t, int i, float &dsc, float &qneg) {
        dsc = h2f(w.d[i]);
        qneg = 0.0f;
    }
    template <int U>
    static __device__ __forceinline__ void read(Raw &w, const uint8_t *blk, uint32_t q) {
#pragma unroll
        for (int s = 0; s < 8; s += 2) {
            w.qs[s] = strip_get4<2>(blk + 18 * s + 2 + 4 * q);
            w.qs[s + 1] = strip_get4<0>(blk + 18 * (s + 1) + 2 + 4 * q);
        }
    }
    static __device__ __forceinline__ long operand(const Raw &w, int s) {
        const uint32_t lo = FmtIQ4XS::lut4(w.qs[s] & 0x0F0F0F0Fu), hi = FmtIQ4XS::lut4((w.qs[s] >> 4) & 0x0F0F0F0Fu);
        return (long)(((uint64_t)hi << 32) | lo);
    }
};

// Q5_0 / Q5_1 in the few-token kernel: lane (c, q) takes bytes 4q..4q+3 of each block's nibbles -- weights 4q..4q+3
// (low nibbles) and 16 + 4q..16 + 4q + 3 (high) -- and their fifth bits, bits 4q.. and 16 + 4q.. of qh; the tokens'
// bytes are staged in that order (ACT_PERM = 2).  Q5_0's fields sit 2 past a dword boundary in the even blocks.
// The "- 16" / "+ m" through the zero-point term.  Strip rows of 92 / 100 dwords: no bank conflicts among the 64
// lanes of a dword read; one token tile (the strips leave LDS for that at two work groups per compute unit).
template <uint32_t TYPE_ID, uint32_t STRIDE, bool WITH_M>
struct SkinnyQ5x {
    static constexpr bool OK = true;
    static constexpr uint32_t BLOCK = 8 * STRIDE, ROW_STRIDE = 2 * BLOCK + 16;
    static constexpr bool HAS_MIN = true, TABLE = true, ONE_TILE = true;
    static constexpr int ACT_PERM = 2, KSPLIT = 1;
    static constexpr uint32_t QH = WITH_M ? 4 : 2;
    struct Raw {
        uint32_t dm[4];
        uint32_t qs[8], qh[8];
    };
    static __device__ __forceinline__ void read_hdr(Raw &w, const uint8_t *blk, uint32_t half) {
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const uint8_t *b = blk + STRIDE * (4 * half + i);
            if constexpr (WITH_M) w.dm[i] = *reinterpret_cast<const uint32_t *>(b);
            else w.dm[i] = reinterpret_cast<const StripR2 *>(b)->v;
        }
    }
    static __device__ __forceinline__ void factors(const Raw &w, uint32_t, int i, float &dsc, float &qneg) {
        dsc = h2f(w.dm[i] & 0xFFFF);
        qneg = WITH_M ? h2f(w.dm[i] >> 16) : -(16.0f * dsc);  // exact
    }
    template <int U>
    static __device__ __forceinline__ void read(Raw &w, const uint8_t *blk, uint32_t q) {
#pragma unroll
        for (int s = 0; s < 8; s++) {
            const uint8_t *b = blk + STRIDE * s;
            if constexpr (WITH_M) {
                w.qh[s] = *reinterpret_cast<const uint32_t *>(b + QH);
                w.qs[s] = *reinterpret_cast<const uint32_t *>(b + QH + 4 + 4 * q);
            } else if (s % 2 == 0) {
                w.qh[s] = strip_get4<2>(b + QH);
                w.qs[s] = strip_get4<2>(b + QH + 4 + 4 * q);
            } else {
                w.qh[s] = strip_get4<0>(b + QH);
                w.qs[s] = strip_get4<0>(b + QH + 4 + 4 * q);
            }
            w.qh[s] >>= 4 * q;  // the lane's fifth bits: bits 0..3 (low nibbles) and 16..19 (high)
        }
    }
    static __device__ __forceinline__ long operand(const Raw &w, int s) {
        const uint32_t lo = (w.qs[s] & 0x0F0F0F0Fu) | (spread4(w.qh[s] & 0xFu) << 4);
        const uint32_t hi = ((w.qs[s] >> 4) & 0x0F0F0F0Fu) | (spread4((w.qh[s] >> 16) & 0xFu) << 4);
        return (long)(((uint64_t)hi << 32) | lo);
    }
};
template <>
struct Skinny<TileQ5_0> : SkinnyQ5x<OXQ_TYPE_Q5_0, 22, false> {};
template <>
struct Skinny<TileQ5_1> : SkinnyQ5x<OXQ_TYPE_Q5_1, 24, true> {};

// The few-token kernel for the formats of this translation unit: the launch shape that serves a call (0: none), and
// the launch.
int skinny_shape_more(uint32_t type, const GemmArgs &a, bool has_partial, uint32_t rows, int variant) {
    switch (type) {
    case OXQ_TYPE_Q5_K: return skinny_shape<TileQ5K>(a, has_partial, rows, variant);
    case OXQ_TYPE_Q3_K: return skinny_shape<TileQ3K>(a, has_partial, rows, variant);
    case OXQ_TYPE_Q4_1: return skinny_shape<TileQ4_1>(a, has_partial, rows, variant);
    case OXQ_TYPE_IQ4_NL: return skinny_shape<TileIQ4NL>(a, has_partial, rows, variant);
    case OXQ_TYPE_Q2_K: return skinny_shape<TileQ2K>(a, has_partial, rows, variant);
    case OXQ_TYPE_Q5_0: return skinny_shape<TileQ5_0>(a, has_partial, rows, variant);
    case OXQ_TYPE_Q5_1: return skinny_shape<TileQ5_1>(a, has_partial, rows, variant);
    default: return (int)SK_NONE;
    }
}
hipError_t launch_skinny_more(uint32_t type, const GemmArgs &a, const TilePlan &plan, hipStream_t stream, int shape) {
    switch (type) {
    case OXQ_TYPE_Q5_K: return launch_skinny<TileQ5K>(a, plan, stream, shape);
    case OXQ_TYPE_Q3_K: return launch_skinny<TileQ3K>(a, plan, stream, shape);
    case OXQ_TYPE_Q4_1: return launch_skinny<TileQ4_1>(a, plan, stream, shape);
    case OXQ_TYPE_IQ4_NL: return launch_skinny<TileIQ4NL>(a, plan, stream, shape);
    case OXQ_TYPE_Q2_K: return launch_skinny<TileQ2K>(a, plan, stream, shape);
    case OXQ_TYPE_Q5_0: return launch_skinny<TileQ5_0>(a, plan, stream, shape);
    case OXQ_TYPE_Q5_1: return launch_skinny<TileQ5_1>(a, plan, stream, shape);
    default: return hipErrorNotSupported;
    }
}

hipError_t launch_tiles_more(uint32_t type, const GemmArgs &a, const TilePlan &plan, hipStream_t stream) {
    switch (type) {
    case OXQ_TYPE_Q5_K: return launch_tiles<TileQ5K>(a, plan, stream);
    case OXQ_TYPE_Q4_1: return launch_tiles<TileQ4_1>(a, plan, stream);
    case OXQ_TYPE_IQ4_NL: return launch_tiles<TileIQ4NL>(a, plan, stream);
    case OXQ_TYPE_Q8_1: return launch_tiles<TileQ8_1>(a, plan, stream);
    case OXQ_TYPE_Q5_0: return launch_tiles<TileQ5_0>(a, plan, stream);
    case OXQ_TYPE_Q5_1: return launch_tiles<TileQ5_1>(a, plan, stream);
    case OXQ_TYPE_Q3_K: return launch_tiles<TileQ3K>(a, plan, stream);
    case OXQ_TYPE_Q2_K: return launch_tiles<TileQ2K>(a, plan, stream);
    default: return hipErrorInvalidValue;
    }
}

}  // namespace oxq
