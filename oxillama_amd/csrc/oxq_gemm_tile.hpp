// Kernel and launch templates of the batched form, shared by the translation units that
// instantiate them for their formats.
//
// Batched (prefill, decode batch, mixture-of-experts group) form of the fused matvec on gfx950:
//   out[m x n] (+)= A_q8[m rows of Q8_0 blocks] x W[n x k]^T
// i.e. m fused matvecs over the same weight blocks (the reference's gemm is exactly
// that loop, crates/oxillama-quant/src/reference/q4_k.rs:186-201, with
// matvec_q8_fused's arithmetic, :218-333), for all five formats.
//
// The contraction runs on the int8 matrix cores.  One v_mfma_i32_32x32x32_i8 contracts one
// 32-weight sub-block of 32 weight rows against the matching Q8_0 block of 32 tokens, so
// every int32 result is exactly one "group sum" I[m][n][s] of the matvec (Q6_K, whose scales
// change every 16 weights, uses two v_mfma_i32_32x32x16_i8 per sub-block).  The fp32 value is
//   y[m][n] = sum_s da[m][s] * dsc[n][s] * I[m][n][s]  +  sum_s (da[m][s]*S[m][s]) * z[n][s]
// with dsc the weight scale of the sub-block (d*sc for the K-quants), S the sum of the block's
// int8 activations and z the zero-point factor (-dmin*mn for Q4_K, -8*d for Q4_0, else absent).
//  * first sum: the MFMA adds into the constant 0x4B400000 (= 12582912.0f), so the
//    int32 result read as a float is 12582912 + I exactly; one fma with the per-lane
//    constants dsc and -12582912*dsc (exact: dsc has <= 19 significant bits) gives
//    fl(dsc * I) -- the rounding of the reference's `da * dot as f32` -- without an
//    int->float conversion, and a second fma with the token's f16 scale accumulates.
//    Two VALU operations per (token, weight row, sub-block): that, not the matrix
//    core, bounds this kernel.
//  * second sum: a rank-(k/32) fp32 product, added into the same accumulators with
//    v_mfma_f32_32x32x2_f32 on P[m][s] = da*S and z while the VALU works on other tiles.
// A small preparation kernel lays the activations out once per call: int8 payload
// tiled [k/32][m][32] in the byte order the format's operands need (so every MFMA operand
// load is one aligned, contiguous KB), P as fp32 [k/32][m], da as f16 [k/32][m].
#pragma once
#include <type_traits>
#include "oxq_gemv_kernel.hpp"
#include "oxq_internal.hpp"

namespace oxq {


typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef float v16f __attribute__((ext_vector_type(16)));

constexpr uint32_t MAGIC_BITS = 0x4B400000u;  // 1.5 * 2^23: float(MAGIC_BITS + i) == 12582912 + i for |i| < 2^22
constexpr float MAGIC_F = 12582912.0f;
constexpr int BUFFER_FLAGS = 0x00020000;  // raw buffer descriptor word 3 on gfx9: 32-bit data format, no swizzle

// ---- per-format pieces of the tile kernel ------------------------------------------------
// 256 consecutive weights of a row (a K-quant super-block, or 8 blocks of the 32-weight
// formats) are walked as 4 groups of 2 sub-blocks of 32 weights; sub-block s meets the
// activation block 8*blk + s.  For each group a lane (c, h) fetches NQ 16-byte pieces of its
// row and turns them into the B operands of the MFMAs of both sub-blocks.  A format says:
//   sub_block(g, e)   which sub-block (0..7) the e-th of group g is
//   fetch             the lane's NQ loads for group g (scalar offset + fixed lane offset)
//   operands          int8 B operands from those bytes: one K = 32 operand per sub-block, or
//                     (KSPLIT = 2, scales every 16 weights) one K = 16 operand per half
//   load_hdr/factors  the fp32 scale factors of a row's sub-blocks: dsc per (sub-block, half)
//                     and, HAS_MIN, the factor of the zero-point term
//   ACT_PERM          the byte order the activations must have so that k-slots line up

typedef long i64x1;

template <int KSPLIT>
struct BOperand;
template <>
struct BOperand<1> {
    v4i k32;  // 16 bytes: k-slots 16h..16h+15 of the sub-block
};
template <>
struct BOperand<2> {
    long k16[2];  // per 16-weight half: 8 bytes, k-slots 8h..8h+7 of the half
};

__device__ __forceinline__ u32x4 buf16(__amdgpu_buffer_rsrc_t rs, uint32_t voff, uint32_t soff) {
    return __builtin_amdgcn_raw_buffer_load_b128(rs, voff, soff, 0);
}
// 16 bytes at an offset that is 2 mod 4 (soff >= 2): an aligned 16-byte load two bytes earlier plus the next
// dword, funnel-shifted.  Sub-dword-misaligned 16-byte loads cost a large part of the load bandwidth.
__device__ __forceinline__ u32x4 buf16_off2(__amdgpu_buffer_rsrc_t rs, uint32_t voff, uint32_t soff) {
    const u32x4 lo = __builtin_amdgcn_raw_buffer_load_b128(rs, voff, soff - 2, 0);
    const uint32_t hi = (uint32_t)__builtin_amdgcn_raw_buffer_load_b32(rs, voff, soff + 14, 0);
    u32x4 r;
    r[0] = __builtin_amdgcn_alignbit(lo[1], lo[0], 16);
    r[1] = __builtin_amdgcn_alignbit(lo[2], lo[1], 16);
    r[2] = __builtin_amdgcn_alignbit(lo[3], lo[2], 16);
    r[3] = __builtin_amdgcn_alignbit(hi, lo[3], 16);
    return r;
}
// The same with the misalignment depending on the lane: 16 bytes starting `shift` / 8 bytes (0 or 2) after the
// dword-aligned offset voff + soff.
__device__ __forceinline__ u32x4 buf16_shift(__amdgpu_buffer_rsrc_t rs, uint32_t voff, uint32_t soff, uint32_t shift) {
    const u32x4 lo = __builtin_amdgcn_raw_buffer_load_b128(rs, voff, soff, 0);
    const uint32_t hi = (uint32_t)__builtin_amdgcn_raw_buffer_load_b32(rs, voff, soff + 16, 0);
    u32x4 r;
    r[0] = __builtin_amdgcn_alignbit(lo[1], lo[0], shift);
    r[1] = __builtin_amdgcn_alignbit(lo[2], lo[1], shift);
    r[2] = __builtin_amdgcn_alignbit(lo[3], lo[2], shift);
    r[3] = __builtin_amdgcn_alignbit(hi, lo[3], shift);
    return r;
}

// Q4_K (reference/q4_k.rs:27-102): 144 B = d, dmin, 12 B of 6-bit scales/mins, 128 B nibbles.
// The lane's 16 bytes qs[32g + 16h ..] carry weights 16h..16h+15 of sub-block 2g in the low
// nibbles and of sub-block 2g+1 in the high nibbles.
struct TileQ4K {
    static constexpr uint32_t TYPE = OXQ_TYPE_Q4_K, BLOCK_BYTES = 144;
    static constexpr bool HAS_MIN = true;
    static constexpr int ACT_PERM = 0, NQ = 1, KSPLIT = 1;
    struct Hdr {
        u32x4 w;  // d | dmin<<16, scales[0..4], [4..8], [8..12]
    };
    static __device__ __forceinline__ uint32_t sub_block(uint32_t g, uint32_t e) { return 2 * g + e; }
    static __device__ __forceinline__ void fetch(__amdgpu_buffer_rsrc_t rs, uint32_t row_off, uint32_t h, uint32_t so_blk,
                                                 uint32_t g, u32x4 (&qs)[NQ]) {
        qs[0] = buf16(rs, row_off + 16 * h, so_blk + 16 + 32 * g);
    }
    template <int SPL>
    static __device__ __forceinline__ void load_hdr(__amdgpu_buffer_rsrc_t rs, uint32_t row_off, uint32_t so_blk, uint32_t,
                                                    Hdr &hd) {
        hd.w = buf16(rs, row_off, so_blk);
    }
    // decode_scales_mins, reference/q4_k.rs:27-49
    static __device__ __forceinline__ void factors(const Hdr &hd, uint32_t, uint32_t s, float (&dsc)[KSPLIT], float &qneg) {
        const uint32_t sh = 8 * (s & 3);
        uint32_t sc, mn;
        if (s < 4) {
            sc = (hd.w[1] >> sh) & 63;
            mn = (hd.w[2] >> sh) & 63;
        } else {
            sc = ((hd.w[3] >> sh) & 15) | (((hd.w[1] >> (sh + 6)) & 3) << 4);
            mn = ((hd.w[3] >> (sh + 4)) & 15) | (((hd.w[2] >> (sh + 6)) & 3) << 4);
        }
        dsc[0] = h2f(hd.w[0] & 0xFFFF) * (float)sc;  // reference/q4_k.rs:280, exact
        qneg = -(h2f(hd.w[0] >> 16) * (float)mn);    // reference/q4_k.rs:281, exact
    }
    static __device__ __forceinline__ void operands(const u32x4 (&qs)[NQ], uint32_t, BOperand<1> (&bop)[2]) {
        for (int i = 0; i < 4; i++) {
            bop[0].k32[i] = (int)(qs[0][i] & 0x0F0F0F0Fu);
            bop[1].k32[i] = (int)((qs[0][i] >> 4) & 0x0F0F0F0Fu);
        }
    }
};

// Swap so that, of two 16-byte pieces held one by each half of the wave (half h holds piece
// h), every lane ends up with bytes 8h..8h+7 of piece 0 (x[0]) and of piece 1 (x[1]).
__device__ __forceinline__ void halves_to_pieces(const u32x4 q, uint32_t (&x)[2][2]) {
    const auto s02 = __builtin_amdgcn_permlane32_swap(q[0], q[2], false, false);
    const auto s13 = __builtin_amdgcn_permlane32_swap(q[1], q[3], false, false);
    x[0][0] = s02[0];
    x[0][1] = s13[0];
    x[1][0] = s02[1];
    x[1][1] = s13[1];
}

// IQ4_XS (reference/iq4_xs.rs:47-97): 136 B = d, scales_h, scales_l, 128 B of indices.  The
// lane's 16 bytes are the whole sub-block 2g+h, byte j = codebook indices of weights 2j (low
// nibble) and 2j+1 (high).  After halves_to_pieces the table lookup yields weights
// 16h + {0,2,4,6, 1,3,5,7, 8,10,12,14, 9,11,13,15}; the preparation kernel stores the
// activation bytes in that same order (ACT_PERM = 1).
struct TileIQ4XS {
    static constexpr uint32_t TYPE = OXQ_TYPE_IQ4_XS, BLOCK_BYTES = 136;
    static constexpr bool HAS_MIN = false;
    static constexpr int ACT_PERM = 1, NQ = 1, KSPLIT = 1;
    struct Hdr {
        u32x4 w;  // d | scales_h<<16, scales_l, (indices)
    };
    static __device__ __forceinline__ uint32_t sub_block(uint32_t g, uint32_t e) { return 2 * g + e; }
    static __device__ __forceinline__ void fetch(__amdgpu_buffer_rsrc_t rs, uint32_t row_off, uint32_t h, uint32_t so_blk,
                                                 uint32_t g, u32x4 (&qs)[NQ]) {
        qs[0] = buf16(rs, row_off + 16 * h, so_blk + 8 + 32 * g);
    }
    template <int SPL>
    static __device__ __forceinline__ void load_hdr(__amdgpu_buffer_rsrc_t rs, uint32_t row_off, uint32_t so_blk, uint32_t,
                                                    Hdr &hd) {
        hd.w = buf16(rs, row_off, so_blk);
    }
    // unpack_sub_scale, reference/iq4_xs.rs:47-53; scale = d * ls first, :81
    static __device__ __forceinline__ void factors(const Hdr &hd, uint32_t, uint32_t s, float (&dsc)[KSPLIT], float &qneg) {
        const uint32_t ls = ((hd.w[1] >> (4 * s)) & 15) | ((((hd.w[0] >> 16) >> (2 * s)) & 3) << 4);
        dsc[0] = h2f(hd.w[0] & 0xFFFF) * (float)((int)ls - 32);  // exact
        qneg = 0.0f;
    }
    static __device__ __forceinline__ void operands(const u32x4 (&qs)[NQ], uint32_t, BOperand<1> (&bop)[2]) {
        uint32_t x[2][2];
        halves_to_pieces(qs[0], x);
        for (int e = 0; e < 2; e++)
            for (int i = 0; i < 2; i++) {
                bop[e].k32[2 * i] = (int)FmtIQ4XS::lut4(x[e][i] & 0x0F0F0F0Fu);
                bop[e].k32[2 * i + 1] = (int)FmtIQ4XS::lut4((x[e][i] >> 4) & 0x0F0F0F0Fu);
            }
    }
};

// Q4_0 (reference/q4_0.rs:22-49): 18 B = d, 16 B of nibbles, byte j = weights 2j (low) and
// 2j+1 (high), each minus 8.  Eight blocks make the 256-weight step.  Same interleave as
// IQ4_XS; the "- 8" goes through the zero-point term: sum (q-8) a = sum q a - 8 sum a.
struct TileQ4_0 {
    static constexpr uint32_t TYPE = OXQ_TYPE_Q4_0, BLOCK_BYTES = 8 * 18;
    static constexpr bool RAGGED_K = true;  // eight independent 32-weight blocks: rows of any whole number of them
    static constexpr bool HAS_MIN = true;
    static constexpr int ACT_PERM = 1, NQ = 1, KSPLIT = 1;
    struct Hdr {
        uint32_t d[8];  // f16 scale bits of the lane's sub-blocks
    };
    static __device__ __forceinline__ uint32_t sub_block(uint32_t g, uint32_t e) { return 2 * g + e; }
    static __device__ __forceinline__ void fetch(__amdgpu_buffer_rsrc_t rs, uint32_t row_off, uint32_t h, uint32_t so_blk,
                                                 uint32_t g, u32x4 (&qs)[NQ]) {
        // block 2g + h, its 16 nibble bytes: at 36g + 2 (half 0: 2 past a dword boundary) or 36g + 20 (half 1: aligned)
        qs[0] = buf16_shift(rs, row_off + 20 * h, so_blk + 36 * g, h ? 0u : 16u);
    }
    template <int SPL>
    static __device__ __forceinline__ void load_hdr(__amdgpu_buffer_rsrc_t rs, uint32_t row_off, uint32_t so_blk,
                                                    uint32_t s0, Hdr &hd) {
#pragma unroll
        for (int e = 0; e < SPL; e++)
            hd.d[e] = (uint32_t)(uint16_t)__builtin_amdgcn_raw_buffer_load_b16(rs, row_off + 18 * (s0 + e), so_blk, 0);
    }
    static __device__ __forceinline__ void factors(const Hdr &hd, uint32_t e, uint32_t, float (&dsc)[KSPLIT], float &qneg) {
        dsc[0] = h2f(hd.d[e]);
        qneg = -(8.0f * dsc[0]);  // exact
    }
    static __device__ __forceinline__ void operands(const u32x4 (&qs)[NQ], uint32_t, BOperand<1> (&bop)[2]) {
        uint32_t x[2][2];
        halves_to_pieces(qs[0], x);
        for (int e = 0; e < 2; e++)
            for (int i = 0; i < 2; i++) {
                bop[e].k32[2 * i] = (int)(x[e][i] & 0x0F0F0F0Fu);
                bop[e].k32[2 * i + 1] = (int)((x[e][i] >> 4) & 0x0F0F0F0Fu);
            }
    }
};

// Q8_0 weights (reference/q8_0.rs:22-47): 34 B = d, 32 int8.  Eight blocks make the
// 256-weight step; the payload is the B operand as it is.
struct TileQ8_0 {
    static constexpr uint32_t TYPE = OXQ_TYPE_Q8_0, BLOCK_BYTES = 8 * 34;
    static constexpr bool RAGGED_K = true;
    static constexpr bool HAS_MIN = false;
    static constexpr int ACT_PERM = 0, NQ = 2, KSPLIT = 1;
    struct Hdr {
        uint32_t d[8];
    };
    static __device__ __forceinline__ uint32_t sub_block(uint32_t g, uint32_t e) { return 2 * g + e; }
    static __device__ __forceinline__ void fetch(__amdgpu_buffer_rsrc_t rs, uint32_t row_off, uint32_t h, uint32_t so_blk,
                                                 uint32_t g, u32x4 (&qs)[NQ]) {
        qs[0] = buf16_off2(rs, row_off + 16 * h, so_blk + 68 * g + 2);  // block 2g: payload at 2 mod 4
        qs[1] = buf16(rs, row_off + 16 * h, so_blk + 68 * g + 36);      // block 2g + 1: payload dword-aligned
    }
    template <int SPL>
    static __device__ __forceinline__ void load_hdr(__amdgpu_buffer_rsrc_t rs, uint32_t row_off, uint32_t so_blk,
                                                    uint32_t s0, Hdr &hd) {
#pragma unroll
        for (int e = 0; e < SPL; e++)
            hd.d[e] = (uint32_t)(uint16_t)__builtin_amdgcn_raw_buffer_load_b16(rs, row_off + 34 * (s0 + e), so_blk, 0);
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

// Q6_K (reference/q6_k.rs:25-75): 210 B = ql[128], qh[64], 16 int8 scales, d.  Scales change
// every 16 weights, so each 32-weight sub-block is two K = 16 MFMAs with their own factor.
// Group g = (half hh = g / 2, pair p = g % 2): ql[64hh + 32p + l] holds, for l = 0..31, the low
// 4 bits of sub-block 4hh + p (low nibble) and of sub-block 4hh + p + 2 (high nibble); their
// upper 2 bits sit in qh[32hh + l] at bit 2p and 2p + 4.  Lane (c, h) fetches ql and qh bytes
// 16h..16h+15 (the 16-weight half h of both sub-blocks); halves_to_pieces hands every lane
// bytes 8h..8h+7 of both halves, which is the k-slot order of the K = 16 operand and of the
// activations as the preparation kernel stores them (ACT_PERM = 2).
struct TileQ6K {
    static constexpr uint32_t TYPE = OXQ_TYPE_Q6_K, BLOCK_BYTES = 210;
    static constexpr bool HAS_MIN = false;
    static constexpr int ACT_PERM = 2, NQ = 2, KSPLIT = 2;
    struct Hdr {
        u32x4 sc;    // 16 int8 scales
        uint32_t d;  // f16 bits
    };
    static __device__ __forceinline__ uint32_t sub_block(uint32_t g, uint32_t e) { return 4 * (g >> 1) + (g & 1) + 2 * e; }
    static __device__ __forceinline__ void fetch(__amdgpu_buffer_rsrc_t rs, uint32_t row_off, uint32_t h, uint32_t so_blk,
                                                 uint32_t g, u32x4 (&qs)[NQ]) {
        qs[0] = buf16(rs, row_off + 16 * h, so_blk + 64 * (g >> 1) + 32 * (g & 1));
        qs[1] = buf16(rs, row_off + 16 * h, so_blk + 128 + 32 * (g >> 1));
    }
    template <int SPL>
    static __device__ __forceinline__ void load_hdr(__amdgpu_buffer_rsrc_t rs, uint32_t row_off, uint32_t so_blk, uint32_t,
                                                    Hdr &hd) {
        hd.sc = buf16(rs, row_off, so_blk + 192);
        hd.d = (uint32_t)(uint16_t)__builtin_amdgcn_raw_buffer_load_b16(rs, row_off, so_blk + 208, 0);
    }
    // scale of half `is` of sub-block s: scales[2s + is] (reference/q6_k.rs:55-72: index 8hh + is + 2j)
    static __device__ __forceinline__ void factors(const Hdr &hd, uint32_t, uint32_t s, float (&dsc)[KSPLIT], float &qneg) {
        const uint32_t pair = hd.sc[s >> 1] >> (16 * (s & 1));
        const float d = h2f(hd.d);
        dsc[0] = d * (float)(int)(int8_t)(pair & 0xFF);         // reference/q6_k.rs:62, exact
        dsc[1] = d * (float)(int)(int8_t)((pair >> 8) & 0xFF);
        qneg = 0.0f;
    }
    static __device__ __forceinline__ void operands(const u32x4 (&qs)[NQ], uint32_t g, BOperand<2> (&bop)[2]) {
        uint32_t l[2][2], hb[2][2];
        halves_to_pieces(qs[0], l);
        halves_to_pieces(qs[1], hb);
        const uint32_t p2 = 2 * (g & 1);
        for (int e = 0; e < 2; e++)
            for (int is = 0; is < 2; is++) {
                uint32_t q[2];
                for (int i = 0; i < 2; i++) {
                    const uint32_t lo = (l[is][i] >> (4 * e)) & 0x0F0F0F0Fu;
                    const uint32_t hi = ((hb[is][i] >> (p2 + 4 * e)) & 0x03030303u) << 4;
                    // q - 32 per byte (0..63 -> -32..31) without carries between bytes
                    q[i] = (((lo | hi) | 0x80808080u) - 0x20202020u) ^ 0x80808080u;
                }
                bop[e].k16[is] = (long)(((uint64_t)q[1] << 32) | q[0]);
            }
    }
};

// One thread per (token, activation block): payload copy in the byte order the format's B
// operands have (PERM 1: even bytes then odd bytes inside each 8; PERM 2: the two 8-byte
// halves of each 16-weight half side by side), P = da * sum(q), da.
// p16 (optional): two more planes, da * sum(q) over the first and the second 16 weights of the
// block, for formats whose zero-point term has 16-weight granularity.
template <int PERM>
__global__ __launch_bounds__(256) void gemm_prep_acts(const uint8_t *__restrict__ A, uint8_t *__restrict__ q8t,
                                                     float *__restrict__ P, uint16_t *__restrict__ da16, uint32_t m,
                                                     uint32_t mpad, uint32_t nsb, float *__restrict__ p16,
                                                     uint32_t nsb_row) {
    const uint32_t idx = blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= mpad * nsb) return;
    // eight consecutive threads take eight consecutive blocks of one token (272 contiguous bytes), the next eight
    // the next token: reads in runs of a token row's bytes, writes in runs of eight tokens (256 bytes) per sub-block.
    // nsb is a multiple of 8 (the tile kernel walks 256 columns at a time); a token row holds nsb_row <= nsb blocks.
    // When the row ends inside the last group of eight, that group is the row's LAST eight blocks (the window the
    // kernel reads its weights through, so that no read leaves the row), and the blocks of it that the group
    // before already covers are written as zeros.
    const uint32_t grp = idx >> 3, t = grp % mpad, j = (grp / mpad) * 8 + (idx & 7);
    const uint32_t shift = nsb - nsb_row, last = nsb - 8;
    const uint32_t src = j >= last ? j - shift : j;
    const bool live = j < last || (idx & 7) >= shift;
    u32x4 q[2] = {{0, 0, 0, 0}, {0, 0, 0, 0}};
    uint32_t dbits = 0;
    if (t < m && live) {
        const uint8_t *blk = A + ((size_t)t * nsb_row + src) * Q8_BLOCK_BYTES;
        dbits = ld2(blk);
        q[0] = ld16(blk + 2);
        q[1] = ld16(blk + 18);
    }
    int s0 = 0, s1 = 0;
    for (int i = 0; i < 4; i++) {
        s0 = sdot4(q[0][i], 0x01010101u, s0);
        s1 = sdot4(q[1][i], 0x01010101u, s1);
    }
    const int s = s0 + s1;
    if (PERM == 2) {  // [half 0 | half 1] x [bytes 0-7 | 8-15] -> bytes 8h..8h+7 of both halves in 16-byte piece h
        const u32x4 x0 = q[0], x1 = q[1];
        q[0] = u32x4{x0[0], x0[1], x1[0], x1[1]};
        q[1] = u32x4{x0[2], x0[3], x1[2], x1[3]};
    }
    if (PERM == 1) {
        for (int hf = 0; hf < 2; hf++) {
            const u32x4 x = q[hf];
            q[hf][0] = __builtin_amdgcn_perm(x[1], x[0], 0x06040200u);
            q[hf][1] = __builtin_amdgcn_perm(x[1], x[0], 0x07050301u);
            q[hf][2] = __builtin_amdgcn_perm(x[3], x[2], 0x06040200u);
            q[hf][3] = __builtin_amdgcn_perm(x[3], x[2], 0x07050301u);
        }
    }
    u32x4 *dst = reinterpret_cast<u32x4 *>(q8t + ((size_t)j * mpad + t) * 32);
    dst[0] = q[0];
    dst[1] = q[1];
    P[(size_t)j * mpad + t] = h2f(dbits) * (float)s;
    if (p16) {
        p16[(size_t)j * mpad + t] = h2f(dbits) * (float)s0;
        p16[((size_t)nsb + j) * mpad + t] = h2f(dbits) * (float)s1;
    }
    da16[(size_t)j * mpad + t] = (uint16_t)dbits;
}

// Zero-point planes of a format: 1 (one factor per 32-weight sub-block, F::factors) unless the policy
// says MIN_PLANES = 2 (one per 16-weight half, F::factors2).
template <class F, class = void> struct tile_min_planes { static constexpr int value = 1; };
template <class F> struct tile_min_planes<F, std::void_t<decltype(F::MIN_PLANES)>> {
    static constexpr int value = F::MIN_PLANES;
};
// Formats made of independent 32-weight blocks (the policy says RAGGED_K) take rows of any whole number of blocks
// (at least eight); the others need whole 256-weight super-blocks.
template <class F, class = void> struct tile_ragged_k { static constexpr bool value = false; };
template <class F> struct tile_ragged_k<F, std::void_t<decltype(F::RAGGED_K)>> {
    static constexpr bool value = F::RAGGED_K;
};
// Sub-blocks the planes of the workspace hold for a row of k weights: whole groups of eight.
__host__ __device__ __forceinline__ uint32_t tile_padded_sub_blocks(uint32_t k) { return (k + 255) / 256 * 8; }
// Byte offset, from the start of the P plane, of the two half-block planes (the workspace holds the
// activation bytes, P, the f16 scales, then the half planes: 32 + 4 + 2 bytes per token block before them).
__host__ __device__ __forceinline__ size_t tile_p16_offset(size_t nsb, size_t mpad) { return nsb * mpad * 6; }

// Work group = 4 waves as WM (tokens) x WN (weight rows); each wave owns MT x NT MFMA tiles
// of 32 x 32: a (32*MT*WM)-token x (32*NT*WN)-row tile per work group.  Lane l: c = l % 32
// is the token (A operand) / weight row (B operand) / output column it feeds, h = l / 32
// the 16-byte half of the 32-byte block.  C layout of the 32x32 MFMAs: register v of lane l
// holds row 8*(v/4) + 4*h + v%4 (token), column c (weight row).
//
// Everything lives in the 256 architectural VGPRs (two waves per SIMD), so MFMA results
// are read by the VALU without accumulator-register copies.  Per super-block each wave
// decodes its rows' 8 sub-block scales once into LDS as ready-made fp32 factors
// (dsc, -12582912*dsc, and for Q4_K -dmin*mn); the f16 token scales of the whole k sit in
// LDS for the life of the work group and enter the accumulate fma as f16 operands.  The
// Q4_K min term is folded into the same accumulators by one fp32 MFMA per tile and pair
// of sub-blocks.  Weight bytes are fetched DIST groups ahead (a ring of registers), token
// bytes one group ahead.
// Work groups are numbered so that the token tiles of one set of weight rows run on the
// same XCD at the same time (ids are dealt round-robin to the 8 XCDs), which turns their
// weight reads into L2 hits.
//
// Grouped form (mixture-of-experts): blockIdx.y = expert; expert e multiplies the token
// rows offsets[e] .. offsets[e+1]-1 by the weights at W + e * w_stride.
template <class F, int MT, int NT, int WM, int DIST, bool DUMP, int ADIST>
__device__ __forceinline__ void gemm_tile_body(
    const uint8_t *__restrict__ W, const uint8_t *__restrict__ q8t, const float *__restrict__ P,
    const uint16_t *__restrict__ da16, float *__restrict__ out, int32_t *__restrict__ sums, uint32_t m, uint32_t mpad,
    uint32_t n, uint32_t k, int accumulate, const float *__restrict__ bias, uint32_t m_tiles, uint32_t n_tiles,
    const int32_t *__restrict__ offsets,
    size_t w_stride) {
    constexpr bool SPLITK = WM == 0;  // the four waves share one tile and each walk a quarter of k
    constexpr int WMX = SPLITK ? 1 : WM, WN = SPLITK ? 1 : 4 / WMX;
    constexpr int WG_TOK = 32 * MT * WMX, WG_ROWS = 32 * NT * WN, MTILES = MT * WMX;
    constexpr int KS = F::KSPLIT;                     // MFMAs (and scale factors) per sub-block
    constexpr int MINP = tile_min_planes<F>::value;    // zero-point factors per sub-block
    constexpr int NP = 2 * KS + (F::HAS_MIN ? MINP : 0);  // fp32 factor planes per sub-block in LDS
    constexpr int W_ROWS = 32 * NT;                   // weight rows of one wave
    constexpr int LPR = 64 / W_ROWS, SPL = 8 / LPR;   // scale decode: lanes per row, sub-blocks per lane
    static_assert(NT <= 2 && DIST >= 1, "tile configuration");
    extern __shared__ uint16_t lds_da[];            // [nsb][MTILES][2 halves][16] f16 token scales
    // [wave][sub-block][KS x dsc, KS x -MAGIC*dsc, zero-point factor][row of the wave]; the split-k
    // reduction at the end reuses the same memory (after a barrier), so that it does not cost occupancy
    constexpr size_t SC_BYTES = sizeof(float) * 4 * 8 * NP * W_ROWS;
    constexpr size_t RED_BYTES = SPLITK ? sizeof(float) * 4 * MT * NT * 16 * 64 : 0;
    __shared__ __align__(16) uint8_t lds_static[SC_BYTES > RED_BYTES ? SC_BYTES : RED_BYTES];
    float (*lds_sc)[8][NP][W_ROWS] = reinterpret_cast<float (*)[8][NP][W_ROWS]>(lds_static);
    // A row that ends inside its last group of eight blocks (formats of independent 32-weight blocks only): the
    // last group is read through the window of the row's last eight blocks, so that no load leaves the row, and
    // the `dead` sub-blocks of that window, which the group before has covered, get zero factors (their token
    // bytes and scales in the workspace are zeros as well).
    constexpr bool RAG = tile_ragged_k<F>::value;
    const uint32_t nsb_row = k / 32, nblk = RAG ? (k + 255) / 256 : k / 256, nsb = nblk * 8, ngrp = nblk * 4;
    const uint32_t dead = nsb - nsb_row;
    const uint32_t tid = threadIdx.x, lane = tid & 63;
    // split k: the wave index as a scalar -- everything derived from it (the wave's k range, hence the scalar
    // offsets of its buffer loads) must be known to be wave-uniform, or every load is wrapped in a waterfall
    // loop.  The other shapes only form lane offsets from it and keep the plain value (measured: the prefill
    // shapes lose a few per cent with the scalar form).
    const uint32_t wave = SPLITK ? (uint32_t)__builtin_amdgcn_readfirstlane((int)(tid >> 6)) : tid >> 6;
    const uint32_t c = lane & 31, h = lane >> 5;
    const uint32_t wm = SPLITK ? 0 : wave % WMX, wn = SPLITK ? 0 : wave / WMX;
    // super-blocks of this wave: all of them, or its quarter
    const uint32_t blk_begin = SPLITK ? wave * nblk / 4 : 0, blk_end = SPLITK ? (wave + 1) * nblk / 4 : nblk;

    const uint32_t xcd = blockIdx.x & 7, loc = blockIdx.x >> 3;
    uint32_t n_tile = (loc / m_tiles) * 8 + xcd, m_tile = loc % m_tiles;
    uint32_t row0 = 0, row_end = m;
    if (offsets) {
        // expert groups: token tiles outermost, so that the tiles past an expert's rows (the grid is
        // sized for the largest group) form one run at the end instead of sitting between live ones
        const uint32_t n_groups = (n_tiles + 7) / 8;
        m_tile = loc / n_groups;
        n_tile = (loc % n_groups) * 8 + xcd;
        row0 = (uint32_t)offsets[blockIdx.y];
        row_end = (uint32_t)offsets[blockIdx.y + 1];
        W += (size_t)blockIdx.y * w_stride;
    }
    if (n_tile >= n_tiles || row0 + m_tile * WG_TOK >= row_end) return;  // whole work group
    const uint32_t m_wg = row0 + m_tile * WG_TOK, n_wg = n_tile * WG_ROWS;
    const uint32_t m_wave = m_wg + wm * (32 * MT), n_wave = n_wg + wn * (32 * NT);

    // Token scales of this work group's tokens, permuted so that the 16 values a lane needs
    // for one MFMA tile are 32 contiguous bytes.
    // One task = 8 consecutive tokens of one sub-block (16 bytes in, two 8-byte pieces out: token
    // r = 8a + 4hh + b of a tile goes to [hh][4a + b]); four tasks per trip, loads before stores.
    {
        constexpr uint32_t CH = WG_TOK / 8;  // 8-token chunks per sub-block
        const uint32_t n_tasks = nsb * CH;
        for (uint32_t base = 0; base < n_tasks; base += 4 * 256) {
            u32x4 v[4];
#pragma unroll
            for (int q = 0; q < 4; q++) {
                const uint32_t task = min(base + q * 256 + tid, n_tasks - 1);
                const uint32_t j = task / CH, ch = task % CH;
                v[q] = ld16(reinterpret_cast<const uint8_t *>(da16 + (size_t)j * mpad + m_wg + 8 * ch));
            }
#pragma unroll
            for (int q = 0; q < 4; q++) {
                const uint32_t task = base + q * 256 + tid;
                if (task < n_tasks) {
                    const uint32_t j = task / CH, ch = task % CH;
                    const uint32_t mt = ch >> 2, a = ch & 3;
                    u32x2 *d0 = reinterpret_cast<u32x2 *>(&lds_da[((j * MTILES + mt) * 2 + 0) * 16 + a * 4]);
                    u32x2 *d1 = reinterpret_cast<u32x2 *>(&lds_da[((j * MTILES + mt) * 2 + 1) * 16 + a * 4]);
                    *d0 = u32x2{v[q][0], v[q][1]};
                    *d1 = u32x2{v[q][2], v[q][3]};
                }
            }
        }
    }

    // Operands come through buffer loads: a wave-uniform descriptor, a fixed 32-bit
    // per-lane offset and a scalar offset that advances with k, so the loop spends no
    // vector instructions on addressing.  Rows past n are clamped for loads and masked
    // at the store.
    const uint32_t row_bytes = RAG ? nsb_row * (F::BLOCK_BYTES / 8) : nblk * F::BLOCK_BYTES;
    const uint32_t last_window = row_bytes - F::BLOCK_BYTES;
    auto blk_off = [&](uint32_t blk) { return RAG ? min(blk * F::BLOCK_BYTES, last_window) : blk * F::BLOCK_BYTES; };
    const uint32_t n_base = min(n_wg, n - 1);
    const size_t w_left = (size_t)(n - n_base) * row_bytes;
    const __amdgpu_buffer_rsrc_t rs_w = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<uint8_t *>(W + (size_t)n_base * row_bytes), 0, (int)min(w_left, (size_t)0x7FFFFFFF), BUFFER_FLAGS);
    const __amdgpu_buffer_rsrc_t rs_a =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<uint8_t *>(q8t), 0, (int)(nsb * mpad * 32), BUFFER_FLAGS);
    const __amdgpu_buffer_rsrc_t rs_p = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<float *>(P), 0, (int)(MINP == 2 ? tile_p16_offset(nsb, mpad) + nsb * mpad * 8 : nsb * mpad * 4),
        BUFFER_FLAGS);

    // Scale decode, per wave for its own rows (no work-group barrier in the k loop): lane ->
    // row lane % W_ROWS, sub-blocks SPL * (lane / W_ROWS) + 0..SPL-1.  The wave writes the
    // factors of the next super-block after its last read of the current ones.
    const uint32_t drow = lane % W_ROWS, ds0 = SPL * (lane / W_ROWS);
    const uint32_t hrow_off = (min(n_wave + drow, n - 1) - n_base) * row_bytes;
    auto decode = [&](const typename F::Hdr &hd, uint32_t blk) {
#pragma unroll
        for (int e = 0; e < SPL; e++) {
            const uint32_t s = ds0 + e;
            float dsc[KS], qneg[MINP];
            if constexpr (MINP == 2)
                F::factors2(hd, e, s, dsc, qneg);
            else
                F::factors(hd, e, s, dsc, qneg[0]);
            if (RAG && blk == nblk - 1 && s < dead) {
                for (int is = 0; is < KS; is++) dsc[is] = 0.0f;
                for (int ip = 0; ip < MINP; ip++) qneg[ip] = 0.0f;
            }
#pragma unroll
            for (int is = 0; is < KS; is++) {
                lds_sc[wave][s][is][drow] = dsc[is];
                lds_sc[wave][s][KS + is][drow] = -(MAGIC_F * dsc[is]);  // exact
            }
            if (F::HAS_MIN)
                for (int ip = 0; ip < MINP; ip++) lds_sc[wave][s][2 * KS + ip][drow] = qneg[ip];
        }
    };
    {
        typename F::Hdr hd;
        F::template load_hdr<SPL>(rs_w, hrow_off, blk_off(min(blk_begin, nblk - 1)), ds0, hd);
        decode(hd, min(blk_begin, nblk - 1));
    }

    v16f acc[MT][NT];
    v16i magic;
    for (int i = 0; i < 16; i++) magic[i] = (int)MAGIC_BITS;
    for (int a = 0; a < MT; a++)
        for (int b = 0; b < NT; b++)
            for (int i = 0; i < 16; i++) acc[a][b][i] = 0.0f;

    uint32_t nrow[NT], wq_off[NT];  // wq_off: byte offset of the lane's row from the descriptor base
    for (int nt = 0; nt < NT; nt++) {
        nrow[nt] = n_wave + nt * 32 + c;
        wq_off[nt] = (min(nrow[nt], n - 1) - n_base) * row_bytes;
    }
    uint32_t aq_off[MT], pq_off[MT];
    for (int mt = 0; mt < MT; mt++) {
        const uint32_t tok = m_wave + mt * 32 + c;  // always < mpad
        aq_off[mt] = tok * 32 + 16 * h;             // the lane's 16 bytes of its token's activation block
        pq_off[mt] = (h * mpad + tok) * 4;          // P of the sub-block the lane's half feeds to the min term
    }

    struct Wq {
        u32x4 q[NT][F::NQ];
    };
    struct Ops {
        u32x4 a[2][MT];  // [sub-block of the pair][token tile] 16 activation bytes
        float pv[MT][MINP];  // P of sub-block sub_block(g, h) (MINP = 2: of its two halves)
    };
    // group index G = 4*blk + g; groups past the end re-read the last one (result unused)
    auto fetch_w = [&](Wq &w, uint32_t G) {
        G = min(G, ngrp - 1);
        for (int nt = 0; nt < NT; nt++) F::fetch(rs_w, wq_off[nt], h, blk_off(G >> 2), G & 3, w.q[nt]);
    };
    auto fetch_a = [&](Ops &o, uint32_t G) {
        G = min(G, ngrp - 1);
        const uint32_t blk8 = (G >> 2) * 8, g = G & 3;
        for (int e = 0; e < 2; e++)
            for (int mt = 0; mt < MT; mt++)
                o.a[e][mt] = buf16(rs_a, aq_off[mt], (blk8 + F::sub_block(g, e)) * mpad * 32);
        if (F::HAS_MIN)
            for (int mt = 0; mt < MT; mt++)  // sub_block(g, 0) and (g, 1) are adjacent for every format with a min term
                for (int ip = 0; ip < MINP; ip++) {
                    const uint32_t plane = MINP == 2 ? (uint32_t)tile_p16_offset(nsb, mpad) + ip * nsb * mpad * 4 : 0u;
                    o.pv[mt][ip] = __builtin_bit_cast(
                        float, __builtin_amdgcn_raw_buffer_load_b32(rs_p, pq_off[mt],
                                                                    plane + (blk8 + F::sub_block(g, 0)) * mpad * 4, 0));
                }
    };

    // One group: 2 sub-blocks x KS MFMAs x MT x NT tiles, each MFMA followed by its 32 VALU
    // operations; the MFMA of tile t+2 is issued before the VALU work of tile t+1 so that the
    // matrix core runs ahead of the VALU.
    auto compute = [&](const Wq &w, const Ops &o, uint32_t blk, uint32_t g) {
        constexpr int T = 2 * KS * MT * NT;
        BOperand<KS> bop[NT][2];
        for (int nt = 0; nt < NT; nt++) F::operands(w.q[nt], g, bop[nt]);
        auto mfma_tile = [&](int t) {
            const int e = t / (KS * MT * NT), is = (t / (MT * NT)) % KS, mt = (t / NT) % MT, nt = t % NT;
            if constexpr (KS == 1) {
                v4i aop;
                for (int i = 0; i < 4; i++) aop[i] = (int)o.a[e][mt][i];
                return __builtin_amdgcn_mfma_i32_32x32x32_i8(aop, bop[nt][e].k32, magic, 0, 0, 0);
            } else {
                const long aop = (long)(((uint64_t)o.a[e][mt][2 * is + 1] << 32) | o.a[e][mt][2 * is]);
                return __builtin_amdgcn_mfma_i32_32x32x16_i8(aop, bop[nt][e].k16[is], magic, 0, 0, 0);
            }
        };
        v16i dq[2];
        dq[0] = mfma_tile(0);
        if (T > 1) dq[1] = mfma_tile(1);
#pragma unroll
        for (int t = 0; t < T; t++) {
            const int e = t / (KS * MT * NT), is = (t / (MT * NT)) % KS, mt = (t / NT) % MT, nt = t % NT;
            const uint32_t s = F::sub_block(g, e), j = blk * 8 + s;
            const float dsc = lds_sc[wave][s][is][nt * 32 + c];
            const float nc2 = lds_sc[wave][s][KS + is][nt * 32 + c];
            const u32x4 *dp = reinterpret_cast<const u32x4 *>(&lds_da[((j * MTILES + wm * MT + mt) * 2 + h) * 16]);
            const u32x4 dav[2] = {dp[0], dp[1]};
            const v16i dres = dq[t & 1];
#pragma unroll
            for (int i = 0; i < 16; i++) {
                const uint32_t dbits = (uint32_t)dres[i];
                // fl(dsc * I), then += * da  (da is an f16 value, exact in fp32)
                const float tt = fmaf(__builtin_bit_cast(float, dbits), dsc, nc2);
                const uint32_t pair = dav[i >> 3][(i >> 1) & 3];
                const float da = h2f((i & 1) ? (pair >> 16) : (pair & 0xFFFF));
                acc[mt][nt][i] = fmaf(tt, da, acc[mt][nt][i]);
                if (DUMP) {
                    const uint32_t row = m_wave + mt * 32 + 8 * (i >> 2) + 4 * h + (i & 3);
                    // (a row's last window: sub-block s of it is block j - dead of the row; dead ones are skipped)
                    const bool shifted = RAG && blk == nblk - 1;
                    if (row < row_end && nrow[nt] < n && !(shifted && s < dead))
                        sums[((size_t)row * n + nrow[nt]) * (nsb_row * KS) + (j - (shifted ? dead : 0)) * KS + is] =
                            (int)(dbits - MAGIC_BITS);
                }
            }
            if (t + 2 < T) dq[t & 1] = mfma_tile(t + 2);
            if (F::HAS_MIN && e == 1 && is == KS - 1) {
                // zero-point term of the group's sub-blocks (lanes h = 0: the first, h = 1: the second):
                // acc[token][row] += P[token][s] * factor[row][s], contracted over the pair
                for (int ip = 0; ip < MINP; ip++) {
                    const float qv = lds_sc[wave][F::sub_block(g, 0) + h][2 * KS + ip][nt * 32 + c];
                    acc[mt][nt] = __builtin_amdgcn_mfma_f32_32x32x2f32(o.pv[mt][ip], qv, acc[mt][nt], 0, 0, 0);
                }
            }
        }
    };

    // Weight ring.  DIST < 4: slot g % DIST is refilled DIST groups ahead as soon as it is consumed.
    // DIST >= 4 (a multiple of 4): ring[i] holds group 4*blk + i; at the top of a super-block the four
    // groups DIST ahead are requested into `incoming`, and the ring advances by four at its end.  The
    // deep form is for few tokens, where the weight stream from HBM paces the kernel and a wave
    // needs many loads in flight.
    constexpr int RING = DIST < 4 ? DIST : DIST;
    static_assert(DIST < 4 || DIST % 4 == 0, "deep prefetch advances by whole super-blocks");
    Wq wring[RING];
    // Token bytes: ring of four slots (slot = group % 4), requested ADIST (1..3) groups ahead.
    static_assert(ADIST >= 1 && ADIST <= 3, "activation prefetch distance");
    Ops ops[4];
#pragma unroll
    for (int d = 0; d < RING; d++) fetch_w(wring[d], blk_begin * 4 + d);
#pragma unroll
    for (int d = 0; d < ADIST; d++) fetch_a(ops[d], blk_begin * 4 + d);
    __syncthreads();

    for (uint32_t blk = blk_begin; blk < blk_end; blk++) {
        const uint32_t nxt = min(blk + 1, nblk - 1);  // last trip: harmless re-read
        Wq incoming[DIST < 4 ? 1 : 4];
        if constexpr (DIST >= 4) {
#pragma unroll
            for (int i = 0; i < 4; i++) fetch_w(incoming[i], blk * 4 + DIST + i);
        }
        typename F::Hdr hd;
        F::template load_hdr<SPL>(rs_w, hrow_off, blk_off(nxt), ds0, hd);
#pragma unroll
        for (int g = 0; g < 4; g++) {
            const Wq w = DIST < 4 ? wring[g % (DIST < 4 ? DIST : 1)] : wring[DIST < 4 ? 0 : g];
            if constexpr (DIST < 4) fetch_w(wring[g % DIST], blk * 4 + g + DIST);  // slot consumed: refill it
            fetch_a(ops[(g + ADIST) % 4], blk * 4 + g + ADIST);
            // keep the requests up here: the instruction scheduler otherwise sinks them to the end of
            // the group's arithmetic (fewer live registers) and the prefetch distance is lost
            __builtin_amdgcn_sched_barrier(0);
            compute(w, ops[g], blk, g);
        }
        if constexpr (DIST >= 4) {
#pragma unroll
            for (int i = 0; i + 4 < DIST; i++) wring[i] = wring[i + 4];
#pragma unroll
            for (int i = 0; i < 4; i++) wring[DIST - 4 + i] = incoming[i];
        }
        __builtin_amdgcn_wave_barrier();  // the wave's reads of this super-block's factors come first
        decode(hd, nxt);
        __builtin_amdgcn_wave_barrier();
    }

    if constexpr (SPLITK) {
        // The four partial tiles meet in LDS; wave w then adds registers 4w..4w+3 of every tile in
        // the fixed order (w0 + w1) + (w2 + w3) and stores them.
        float (*lds_red)[MT * NT][16][64] = reinterpret_cast<float (*)[MT * NT][16][64]>(lds_static);
        __syncthreads();  // every wave is done with its scale factors
        for (int mt = 0; mt < MT; mt++)
            for (int nt = 0; nt < NT; nt++)
#pragma unroll
                for (int i = 0; i < 16; i++) lds_red[wave][mt * NT + nt][i][lane] = acc[mt][nt][i];
        __syncthreads();
        for (int mt = 0; mt < MT; mt++)
            for (int nt = 0; nt < NT; nt++) {
                if (nrow[nt] >= n) continue;
#pragma unroll
                for (int ii = 0; ii < 4; ii++) {
                    const uint32_t i = 4 * wave + ii;  // register index: rows 8*wave + 4*h + ii
                    const uint32_t row = m_wave + mt * 32 + 8 * wave + 4 * h + ii;
                    if (row < row_end) {
                        const int tl = mt * NT + nt;
                        const float y = (lds_red[0][tl][i][lane] + lds_red[1][tl][i][lane]) +
                                        (lds_red[2][tl][i][lane] + lds_red[3][tl][i][lane]);
                        float *o = out + (size_t)row * n + nrow[nt];
                        *o = accumulate ? *o + y : bias ? y + bias[nrow[nt]] : y;
                    }
                }
            }
        return;
    }
    for (int mt = 0; mt < MT; mt++)
        for (int nt = 0; nt < NT; nt++) {
            if (nrow[nt] >= n) continue;
#pragma unroll
            for (int i = 0; i < 16; i++) {
                const uint32_t row = m_wave + mt * 32 + 8 * (i >> 2) + 4 * h + (i & 3);
                if (row < row_end) {
                    float *o = out + (size_t)row * n + nrow[nt];
                    *o = accumulate ? *o + acc[mt][nt][i] : bias ? acc[mt][nt][i] + bias[nrow[nt]] : acc[mt][nt][i];
                }
            }
        }
}

// The kernel proper, compiled for a fixed number of waves per SIMD (OCC = 2: up to 256 VGPRs,
// OCC = 3: up to 168): the register budget decides how far the compiler lets loads and MFMAs
// run ahead of their use.
#define OXQ_TILE_KERNEL(NAME, OCC)                                                                                   \
    template <class F, int MT, int NT, int WM, int DIST, bool DUMP, int ADIST>                                      \
    __global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(OCC, OCC))) void NAME(                      \
        const uint8_t *__restrict__ W, const uint8_t *__restrict__ q8t, const float *__restrict__ P,                \
        const uint16_t *__restrict__ da16, float *__restrict__ out, int32_t *__restrict__ sums, uint32_t m,         \
        uint32_t mpad, uint32_t n, uint32_t k, int accumulate, const float *__restrict__ bias, uint32_t m_tiles,   \
        uint32_t n_tiles, const int32_t *__restrict__ offsets, size_t w_stride) {                                   \
        gemm_tile_body<F, MT, NT, WM, DIST, DUMP, ADIST>(W, q8t, P, da16, out, sums, m, mpad, n, k, accumulate,     \
                                                         bias, m_tiles, n_tiles, offsets, w_stride);                \
    }
OXQ_TILE_KERNEL(gemm_tile_kernel, 2)
OXQ_TILE_KERNEL(gemm_tile_kernel_occ3, 3)
#undef OXQ_TILE_KERNEL

struct TilePlan {
    const uint8_t *q8t;
    const float *P;
    const uint16_t *da16;
    uint32_t mpad;
    float *partial = nullptr;  // room for the few-token kernel's per-split sums (one matrix, k split), or null
};
// The formats instantiated in the second translation unit, and the activation byte order they need.
hipError_t launch_tiles_more(uint32_t type, const GemmArgs &a, const TilePlan &plan, hipStream_t stream);
int skinny_shape_more(uint32_t type, const GemmArgs &a, bool has_partial, uint32_t rows, int variant);
hipError_t launch_skinny_more(uint32_t type, const GemmArgs &a, const TilePlan &plan, hipStream_t stream, int shape);
int tile_act_perm_more(uint32_t type);
bool tile_needs_p16_more(uint32_t type);

template <class F, int MT, int NT, int WM, int DIST, bool DUMP, int OCC = 2, int ADIST = 1>
static hipError_t launch_tile(const GemmArgs &a, const TilePlan &p, hipStream_t stream) {
    constexpr uint32_t WG_TOK = 32 * MT * (WM ? WM : 1), WG_ROWS = 32 * NT * (WM ? 4 / WM : 1);
    const uint32_t rows = a.offsets ? a.max_rows : a.m;
    const uint32_t m_tiles = (rows + WG_TOK - 1) / WG_TOK, n_tiles = (a.n + WG_ROWS - 1) / WG_ROWS;
    const dim3 grid(8 * ((n_tiles + 7) / 8) * m_tiles, a.offsets ? a.n_experts : 1);
    const size_t lds = (size_t)tile_padded_sub_blocks(a.k) * WG_TOK * 2;
    auto kern = &gemm_tile_kernel<F, MT, NT, WM, DIST, DUMP, ADIST>;
    if constexpr (OCC == 3) kern = &gemm_tile_kernel_occ3<F, MT, NT, WM, DIST, DUMP, ADIST>;
    if (lds > 32 * 1024) {  // beyond the default dynamic LDS limit: opt in (up to the 160 KB of a CU)
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kern),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (e != hipSuccess) return e;
    }
    note_launch(OCC == 3 ? "gemm_tile_kernel_occ3" : "gemm_tile_kernel", F::TYPE, MT, NT, WM, DIST, grid.x, grid.y, 256);
    hipLaunchKernelGGL(kern, grid, dim3(256), lds, stream, a.W, p.q8t, p.P, p.da16, a.out, a.sums, a.m, p.mpad, a.n,
                       a.k, a.accumulate, a.bias, m_tiles, n_tiles, a.offsets, a.w_stride);
    return hipGetLastError();
}

// Tile shape by use: many tokens (prefill) take 128-token work-group tiles; few tokens (a
// mixture-of-experts group, a short prompt, a decode batch) take 32-token tiles with the
// weight bytes fetched further ahead, because that case is paced by the weight stream.
template <class F>
static hipError_t launch_tiles(const GemmArgs &a, const TilePlan &p, hipStream_t stream) {
    uint32_t rows = a.offsets ? (a.shape_rows ? a.shape_rows : a.max_rows) : a.m;
    // Expert groups whose sizes only the device knows (the launch is shaped for twice the mean, the grid covers the
    // worst case): the tile follows the mean -- a larger group takes more tiles, while a tile twice the usual group
    // is half empty everywhere.  8 experts of 14336 x 4096 / 4096 x 14336, IQ4_XS, 12..25 rows each: 108 / 108 us on
    // 32-token tiles against 152 / 164 on 64-token ones; 24..42 rows 136 / 140 against 155 / 167; 38..63 rows on
    // 64 x 32 split-k tiles 163 / 172 against 159 / 258 on 64 x 128.
    // (a mean of 49..64 rows spills over 64 in half the groups: the shapes for 65 rows and more; 256 tokens on those
    // experts 743 us per layer against 781)
    if (a.offsets && a.n_experts && a.shape_rows && a.shape_rows < a.max_rows) {
        const uint32_t mean = (a.m + a.n_experts - 1) / a.n_experts;
        rows = mean > 48 && mean < 65 ? 65 : mean;
    }
    const int variant = g_gemm_variant.load(std::memory_order_relaxed);
    (void)variant;  // (read by the fixed-shape knobs, which the second translation unit leaves out)
    // The f16 token scales of a work group's tokens for the whole k sit in LDS (k / 32 * 2 bytes per token): 128-token
    // tiles up to k = 16384, 64-token tiles up to 32768, 32-token tiles beyond (up to 65536).
    const uint32_t nsb_pad = tile_padded_sub_blocks(a.k);
    const bool fits128 = (size_t)nsb_pad * 256 <= 128 * 1024, fits64 = (size_t)nsb_pad * 128 <= 128 * 1024;
    // more than 384 tokens on a matrix so narrow that even 128 x 64 tiles leave compute units without one (the key /
    // value projections of grouped-query attention): the 64 x 32 split-k tiles of the mid range -- 1024 x 4096 at
    // 512 / 1024 tokens 20.7 / 30.7 us against 45.7 / 49.0, 1024 x 8192 Q8_0 35.7 against 98.9, 3072 x 3072 30.7
    // against 38.5; from one tile per compute unit on (1024 x 4096, 2048 tokens) a tie
    const bool narrow = rows > 384 && fits128 &&
                        (size_t)((rows + 127) / 128) * ((a.n + 63) / 64) * (a.offsets ? a.n_experts : 1) < (size_t)device_cus();
    const bool big = rows > 384 && fits128 && !narrow;
    const bool mid = !big && rows > 64 && fits64;
    // 65..384 tokens (more where k is too long for the 128-token tiles): 64 x 128 tiles (a wave per 32 weight rows)
    // where they give the chip 1.75 work groups per compute
    // unit, else 64 x 32 tiles whose four waves split k -- four times the work groups.  Measured (us, the first
    // against the second): 4096 x 14336, 128 / 256 / 384 tokens, Q4_K 131 / 136 / 143 against 47 / 87 / 127, Q6_K
    // 196 / 198 / 206 against 66 / 125 / 183; 4096 x 4096 Q4_K 44 / 45 / 48 against 19 / 27 / 37, Q8_0 51 / 51 / 54
    // against 21 / 33 / 46; 14336 x 4096 Q4_K 128 / 192 tokens 49 / 70 against 45 / 63, 256 a tie, 384 108 against 113.
    const bool mid_split_k = mid && (narrow || (size_t)((rows + 63) / 64) * ((a.n + 127) / 128) * (a.offsets ? a.n_experts : 1) * 4 <
                                                   7 * (size_t)device_cus());
    if (a.sums)  // debug dump: the same tile layout (and fp32 summation order) as the production choice below
        return big   ? launch_tile<F, 2, 1, 2, 1, true>(a, p, stream)
               : mid ? (mid_split_k ? launch_tile<F, 2, 1, 0, 2, true, 2, 2>(a, p, stream)
                                    : launch_tile<F, 2, 1, 1, 2, true>(a, p, stream))
               : (rows > 32 && fits64) ? launch_tile<F, 2, 1, 0, 2, true, 2, 2>(a, p, stream)
                                       : launch_tile<F, 1, 2, 0, 2, true, 2, 2>(a, p, stream);
#ifndef OXQ_TILE_DEFAULT_SHAPES_ONLY
    switch (variant) {
    case 1: return launch_tile<F, 2, 1, 2, 1, false>(a, p, stream);
    case 3: return launch_tile<F, 2, 2, 2, 1, false>(a, p, stream);
    case 4: return launch_tile<F, 2, 2, 2, 2, false>(a, p, stream);
    case 5: return launch_tile<F, 2, 1, 2, 1, false, 3>(a, p, stream);
    case 6: return launch_tile<F, 4, 1, 1, 2, false>(a, p, stream);
    case 7: return launch_tile<F, 4, 1, 1, 1, false>(a, p, stream);
    case 8: return launch_tile<F, 2, 2, 2, 2, false>(a, p, stream);
    case 12: return launch_tile<F, 1, 2, 1, 2, false>(a, p, stream);
    case 13: return launch_tile<F, 1, 2, 1, 4, false>(a, p, stream);
    case 14: return launch_tile<F, 1, 1, 1, 2, false>(a, p, stream);
    case 16: return launch_tile<F, 2, 1, 1, 2, false>(a, p, stream);
    case 21: return launch_tile<F, 1, 1, 0, 2, false, 2, 2>(a, p, stream);
    case 22: return launch_tile<F, 1, 2, 0, 2, false, 2, 2>(a, p, stream);
    case 23: return launch_tile<F, 2, 1, 0, 2, false, 2, 2>(a, p, stream);
    default: break;
    }
#endif
    {
        // Measured on MI355X at 14336 x 4096 (Q4_K, Q6_K) and on the 8-expert IQ4_XS shapes: up to 64
        // tokens the four waves of a work group share one tile and split k (most work groups, shortest
        // dependency chain per wave); up to 384 tokens 64 x 128 tiles (64 x 32 with k split where those are too
        // few); beyond that 128 x 64 tiles at three waves per SIMD.
        if (big) {
            // 128 x 128 tiles (two waves per SIMD, weight bytes fetched two steps ahead) where they still give the
            // chip one and a half work groups per compute unit: 14336 x 4096, 512 tokens 123 us against 125 us,
            // 2048 tokens 383 us against 422 us; 4096 x 14336 has too few such tiles (214 us against 140 us)
            const size_t wgs = (size_t)((rows + 127) / 128) * ((a.n + 127) / 128) * (a.offsets ? a.n_experts : 1);
            // Within the 128 x 128 tile a wave takes 128 tokens x 32 rows (four token tiles against ONE weight-row
            // tile) rather than 64 x 64: half the weight loads per MFMA, and those are the loads in which every lane
            // reads its own row.  Same bits.  512 x 14336 x 4096: Q8_0 122 us against 158, Q4_0 122 against 141,
            // IQ4_XS 107 against 118, Q6_K 168 against 189; 2048 tokens: Q8_0 388 against 503.  Q4_K, whose weight
            // loads are the lightest per MFMA, is the exception (114 against 111) and keeps 64 x 64.
            constexpr bool wide = F::TYPE != OXQ_TYPE_Q4_K;
            // ... or where the 128 x 64 tiles below would come to between one and two per compute unit: a compute unit
            // with two of them takes twice as long as one with one, so 129..256 of the larger tiles, one per compute
            // unit, finish first (4096 x 14336, 768 tokens: Q8_0 248 us against 348, Q6_K 339 against 397, Q4_K 228
            // against 266; 1024 tokens Q6_K 368 against 421)
            const size_t cus = device_cus();
            // (Q4_K on rows of 4096 columns is the exception: 4096 x 4096, 768 / 1024 tokens 72 / 77 us against 76 / 82)
            if (2 * wgs >= 3 * cus || (2 * wgs > cus && wgs <= cus && (wide || a.k >= 8192)))
                return wide ? launch_tile<F, 4, 1, 1, 1, false>(a, p, stream) : launch_tile<F, 2, 2, 2, 2, false>(a, p, stream);
            // one to one and a half work groups per compute unit: still the better shape for the formats of a
            // byte and more per weight (512 x 8192 x 8192 Q8_0: 149 us against 180)
            if (wide && F::BLOCK_BYTES >= 256 && wgs >= (size_t)device_cus()) return launch_tile<F, 4, 1, 1, 1, false>(a, p, stream);
            return launch_tile<F, 2, 1, 2, 1, false, 3>(a, p, stream);
        }
        if (mid)
            return mid_split_k ? launch_tile<F, 2, 1, 0, 2, false, 2, 2>(a, p, stream) : launch_tile<F, 2, 1, 1, 2, false>(a, p, stream);
        // split k; 64 weight rows (or 64 tokens) per work group only where that still leaves every
        // compute unit at least one work group, else 32 x 32
        const size_t groups = a.offsets ? a.n_experts : 1;
        // 33..64 tokens: one 64-token tile where 32-row tiles still give every compute unit a work group
        // (14336 x 4096, 64 rows: 26.6 us against 31.1 with 32 x 32 tiles; 4096 rows: 61 against 50)
        if (rows > 32 && fits64 && (size_t)((a.n + 31) / 32) * groups >= device_cus())
            return launch_tile<F, 2, 1, 0, 2, false, 2, 2>(a, p, stream);
        if ((size_t)((a.n + 63) / 64) * groups < device_cus())
            return launch_tile<F, 1, 1, 0, 2, false, 2, 2>(a, p, stream);
        if (rows > 32 && fits64) return launch_tile<F, 2, 1, 0, 2, false, 2, 2>(a, p, stream);
        // (also: any number of tokens on rows of more than 32768 columns)
        return launch_tile<F, 1, 2, 0, 2, false, 2, 2>(a, p, stream);
    }
}

}  // namespace oxq
