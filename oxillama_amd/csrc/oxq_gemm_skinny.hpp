// Few tokens per weight matrix (a mixture-of-experts group of up to 32 token rows, a decode batch of up to 16 on one
// matrix): the batched fused matvec
//   out[m x n] (+)= A_q8[m rows of Q8_0 blocks] x W[n x k]^T
// (the reference's gemm loop over matvec_q8_fused, crates/oxillama-quant/src/reference/q4_k.rs:186-201, :218-333)
// built around what the counters say bounds the tile kernel in this case: not HBM, not the matrix core, but the
// texture unit -- every lane of a weight load reads its own row (64 separate accesses per instruction), and the
// token bytes are fetched again by every work group.
//
//  * Weights: a wave owns NT tiles of 16 weight rows.  It reads them as contiguous runs -- consecutive lanes take
//    consecutive 16-byte pieces of a row's two next super-blocks -- into registers, one step ahead, and from there
//    into a private strip of LDS; the lanes then pick their B operands out of LDS in the matrix core's layout.  No
//    barrier: the strip belongs to one wave, whose LDS operations execute in order.
//  * Tokens: the work group copies the Q8_0 bytes, scales and block sums of its (at most 32) tokens for a chunk of
//    k into LDS, already in operand order (straight from the caller's Q8_0 rows: no re-layout launch); all waves
//    read them from there.
//  * v_mfma_i32_16x16x32_i8 with the tokens as the A operand (16 tokens x 32 k) and the weights as B (32 k x 16
//    rows): lane l = (c = l % 16, q = l / 16) supplies k-values 8q..8q+7 of token c and of weight row c and
//    receives the sums of row c against tokens 4q..4q+3.  All of a lane's results belong to one weight row, so its
//    weight-side factor is one value per sub-block (decoded once per step by the wave, kept in a small LDS table).
// Arithmetic per result as in the tile kernel (oxq_gemm_tile.hpp): fl(dsc * isum) by the 1.5 * 2^23 trick, then
// one fma with the token's scale; the zero-point term (Q4_K) as a 16 x 16 x 4 fp32 MFMA per four sub-blocks over
// P = d_a * sum(q_a) and the rows' -dmin * mn.
#pragma once
#include "oxq_gemm_tile.hpp"

namespace oxq {

typedef int v4i32 __attribute__((ext_vector_type(4)));

template <class F>
struct Skinny {
    static constexpr bool OK = false;
};

// Q4_K (reference/q4_k.rs:27-99,218-333): 144 B = d, dmin, 12 B of scales / mins, 4 runs of 32 bytes whose low
// nibbles are sub-block 2g and high nibbles sub-block 2g + 1.  Lane (c, q) takes bytes 8q..8q+7 of each run.
template <>
struct Skinny<TileQ4K> {
    static constexpr bool OK = true;
    static constexpr uint32_t BLOCK = 144, ROW_STRIDE = 304;  // LDS bytes per row of a step (2 blocks + pad)
    static constexpr bool HAS_MIN = true, TABLE = true, ONE_TILE = false;
    static constexpr int ACT_PERM = 0, KSPLIT = 1;
    struct Raw {
        u32x4 hdr;
        u32x2 qs[4];
    };
    static __device__ __forceinline__ void read_hdr(Raw &w, const uint8_t *blk, uint32_t) {
        w.hdr = *reinterpret_cast<const u32x4 *>(blk);
    }
    template <int U>
    static __device__ __forceinline__ void read(Raw &w, const uint8_t *blk, uint32_t q) {
#pragma unroll
        for (int g = 0; g < 4; g++) w.qs[g] = *reinterpret_cast<const u32x2 *>(blk + 16 + 32 * g + 8 * q);
    }
    static __device__ __forceinline__ long operand(const Raw &w, int s) {
        const u32x2 v = w.qs[s >> 1];
        const uint32_t lo = (s & 1) ? (v[0] >> 4) & 0x0F0F0F0Fu : v[0] & 0x0F0F0F0Fu;
        const uint32_t hi = (s & 1) ? (v[1] >> 4) & 0x0F0F0F0Fu : v[1] & 0x0F0F0F0Fu;
        return (long)(((uint64_t)hi << 32) | lo);
    }
    // factors of sub-block 4 * half + i
    static __device__ __forceinline__ void factors(const Raw &w, uint32_t half, int i, float &dsc, float &qneg) {
        TileQ4K::Hdr hd;
        hd.w = w.hdr;
        float d1[1];
        TileQ4K::factors(hd, 0, 4 * half + i, d1, qneg);
        dsc = d1[0];
    }
};

// IQ4_XS (reference/iq4_xs.rs:47-97): 136 B = d, scales_h, scales_l, 8 pieces of 16 bytes, one per sub-block, byte
// j = codebook indices of weights 2j (low nibble) and 2j + 1 (high).  Lane (c, q) takes bytes 4q..4q+3 of each
// piece: weights 8q + {0,2,4,6} from the low nibbles, 8q + {1,3,5,7} from the high ones -- the order the
// preparation kernel gives the token bytes for this format (even bytes, then odd bytes, inside each 8).
template <>
struct Skinny<TileIQ4XS> {
    static constexpr bool OK = true;
    // 272 bytes = 68 dwords per row: lane (c, q) reads dword 68 c + q + const, bank 4 c + q -- all 64 distinct
    static constexpr uint32_t BLOCK = 136, ROW_STRIDE = 272;
    static constexpr bool HAS_MIN = false, TABLE = true, ONE_TILE = false;
    static constexpr int ACT_PERM = 1, KSPLIT = 1;
    struct Raw {
        u32x2 hdr;
        uint32_t qs[8];
    };
    static __device__ __forceinline__ void read_hdr(Raw &w, const uint8_t *blk, uint32_t) {
        w.hdr = *reinterpret_cast<const u32x2 *>(blk);
    }
    template <int U>
    static __device__ __forceinline__ void read(Raw &w, const uint8_t *blk, uint32_t q) {
#pragma unroll
        for (int s = 0; s < 8; s++) w.qs[s] = *reinterpret_cast<const uint32_t *>(blk + 8 + 16 * s + 4 * q);
    }
    static __device__ __forceinline__ long operand(const Raw &w, int s) {
        const uint32_t lo = FmtIQ4XS::lut4(w.qs[s] & 0x0F0F0F0Fu);
        const uint32_t hi = FmtIQ4XS::lut4((w.qs[s] >> 4) & 0x0F0F0F0Fu);
        return (long)(((uint64_t)hi << 32) | lo);
    }
    static __device__ __forceinline__ void factors(const Raw &w, uint32_t half, int i, float &dsc, float &qneg) {
        TileIQ4XS::Hdr hd;
        hd.w = u32x4{w.hdr[0], w.hdr[1], 0, 0};
        float d1[1];
        TileIQ4XS::factors(hd, 0, 4 * half + i, d1, qneg);
        dsc = d1[0];
    }
};

// LDS accesses of the strip at less than their natural alignment (the formats whose fields sit at odd multiples of 2)
struct __attribute__((packed, aligned(8), may_alias)) StripR8 { u32x2 v; };
struct __attribute__((packed, aligned(4), may_alias)) StripR4 { uint32_t v; };
struct __attribute__((packed, aligned(2), may_alias)) StripR2 { uint16_t v; };
// 8 bytes at p, which is MIS (0, 2, 4, 6) past a multiple of 8.  2 or 6 past: the three dwords from p - 2 on (an
// aligned 8 bytes and a dword, in this order or the other), funnel-shifted; 4 past: two dwords as they are
template <int MIS>
__device__ __forceinline__ u32x2 strip_get8(const uint8_t *p) {
    if constexpr (MIS == 0) {
        return reinterpret_cast<const StripR8 *>(p)->v;
    } else if constexpr (MIS == 4) {
        return u32x2{reinterpret_cast<const StripR4 *>(p)->v, reinterpret_cast<const StripR4 *>(p + 4)->v};
    } else if constexpr (MIS == 2) {
        const u32x2 lo = reinterpret_cast<const StripR8 *>(p - 2)->v;
        const uint32_t hi = reinterpret_cast<const StripR4 *>(p + 6)->v;
        return u32x2{__builtin_amdgcn_alignbit(lo[1], lo[0], 16), __builtin_amdgcn_alignbit(hi, lo[1], 16)};
    } else {
        const uint32_t lo = reinterpret_cast<const StripR4 *>(p - 2)->v;
        const u32x2 hi = reinterpret_cast<const StripR8 *>(p + 2)->v;
        return u32x2{__builtin_amdgcn_alignbit(hi[0], lo, 16), __builtin_amdgcn_alignbit(hi[1], hi[0], 16)};
    }
}
// 4 bytes at p, MIS (0 or 2) past a multiple of 4
template <int MIS>
__device__ __forceinline__ uint32_t strip_get4(const uint8_t *p) {
    if constexpr (MIS == 0) {
        return reinterpret_cast<const StripR4 *>(p)->v;
    } else {
        return __builtin_amdgcn_alignbit(reinterpret_cast<const StripR4 *>(p + 2)->v, reinterpret_cast<const StripR4 *>(p - 2)->v, 16);
    }
}

// Q4_0 (reference/q4_0.rs:22-49): 18 B = d, 16 bytes of nibbles, byte j = weights 2j (low) and 2j + 1 (high), each
// minus 8.  Eight blocks (144 B) stand for a super-block.  Lane (c, q) takes bytes 4q..4q+3 of each block, as for
// IQ4_XS; they sit 2 past a dword boundary in the even blocks.  The operand is the unsigned nibble; the "- 8" goes
// through the zero-point term (P times -8 d), as in the tile kernel.
template <>
struct Skinny<TileQ4_0> {
    static constexpr bool OK = true;
    static constexpr uint32_t BLOCK = 144, ROW_STRIDE = 304;
    static constexpr bool HAS_MIN = true, TABLE = true, ONE_TILE = false;
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
        qneg = -(8.0f * dsc);  // exact
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
        const uint32_t lo = w.qs[s] & 0x0F0F0F0Fu, hi = (w.qs[s] >> 4) & 0x0F0F0F0Fu;
        return (long)(((uint64_t)hi << 32) | lo);
    }
};

// Q8_0 weights (reference/q8_0.rs:22-47): 34 B = d, 32 int8, the operand as it is.  Eight blocks (272 B) stand for a
// super-block; a row's step is 544 bytes, and the strip rows are packed at that stride: with it, the token bytes
// of a chunk of two super-blocks and no factor table, two work groups still share a compute unit's LDS.  The
// scale is read from the strip with the block's bytes.  Lane (c, q) takes payload bytes 8q..8q+7, which sit 2, 4, 6
// or 0 bytes past a multiple of 8 as the block index goes up.
template <>
struct Skinny<TileQ8_0> {
    static constexpr bool OK = true;
    static constexpr uint32_t BLOCK = 272, ROW_STRIDE = 544;
    static constexpr bool HAS_MIN = false, TABLE = false, ONE_TILE = true;
    static constexpr int ACT_PERM = 0, KSPLIT = 1;
    struct Raw {
        uint32_t d[8];
        u32x2 qs[8];
    };
    template <int U>
    static __device__ __forceinline__ void read(Raw &w, const uint8_t *blk, uint32_t q) {
#pragma unroll
        for (int s = 0; s < 8; s += 4) {
            w.qs[s] = strip_get8<2>(blk + 34 * s + 2 + 8 * q);
            w.qs[s + 1] = strip_get8<4>(blk + 34 * (s + 1) + 2 + 8 * q);
            w.qs[s + 2] = strip_get8<6>(blk + 34 * (s + 2) + 2 + 8 * q);
            w.qs[s + 3] = strip_get8<0>(blk + 34 * (s + 3) + 2 + 8 * q);
        }
#pragma unroll
        for (int s = 0; s < 8; s++) w.d[s] = reinterpret_cast<const StripR2 *>(blk + 34 * s)->v;
    }
    static __device__ __forceinline__ long operand(const Raw &w, int s) {
        return (long)(((uint64_t)w.qs[s][1] << 32) | w.qs[s][0]);
    }
    static __device__ __forceinline__ float scale(const Raw &w, int s) { return h2f(w.d[s]); }
};

// Q6_K (reference/q6_k.rs:25-75): 210 B = ql[128], qh[64], 16 int8 scales, d.  Sub-block s = 4 hh + p + 2 e of 32
// weights has its low 4 bits in ql[64 hh + 32 p + l] (low nibble e = 0, high nibble e = 1) and its upper 2 bits in
// qh[32 hh + l] at bit 2 p + 4 e; its two halves of 16 weights have their own scales, scales[2 s] and [2 s + 1].
// Lane (c, q) takes weights 8q..8q+7 of every sub-block: 8 bytes of ql per (hh, p), 8 of qh per hh.
//  * The step's second block starts 210 bytes into the row's strip: 2 past a multiple of 8.  Its fields are read as
//    the aligned 8 bytes below plus the next dword, funnel-shifted.
//  * One MFMA per half: the lanes of the other half (q / 2) supply zeros.  Each half's result is scaled by its own
//    factor, as the reference scales 16 weights at a time (q6_k.rs:62-70).
//  * The operand is q (0..63), not q - 32: the MFMA's addend carries -32 * sum of the token's 16 activations
//    (integers, exact), so the result is the reference's sum of (q - 32) * a.
template <>
struct Skinny<TileQ6K> {
    static constexpr bool OK = true;
    // 432 bytes = 108 dwords per row: rows start on multiples of 16 bytes
    static constexpr uint32_t BLOCK = 210, ROW_STRIDE = 432;
    static constexpr bool HAS_MIN = false, TABLE = true, ONE_TILE = true;
    static constexpr int ACT_PERM = 0, KSPLIT = 2, OFFSET = 32;
    struct Raw {
        u32x2 ql[4], qh[2];
    };
    // U: the step's first block (fields on multiples of 8) or its second (2 past)
    template <int U>
    static __device__ __forceinline__ void read(Raw &w, const uint8_t *blk, uint32_t q) {
#pragma unroll
        for (int g = 0; g < 4; g++) w.ql[g] = strip_get8<2 * U>(blk + 32 * g + 8 * q);
#pragma unroll
        for (int hh = 0; hh < 2; hh++) w.qh[hh] = strip_get8<2 * U>(blk + 128 + 32 * hh + 8 * q);
    }
    static __device__ __forceinline__ long operand(const Raw &w, int s) {
        const int hh = s >> 2, p = s & 1, e = (s >> 1) & 1, sh = 2 * p + 4 * e;
        const u32x2 l = w.ql[2 * hh + p], h = w.qh[hh];
        uint32_t v[2];
#pragma unroll
        for (int i = 0; i < 2; i++) {
            const uint32_t lo = e ? (l[i] >> 4) & 0x0F0F0F0Fu : l[i] & 0x0F0F0F0Fu;
            const uint32_t hs = sh < 4 ? h[i] << (4 - sh) : h[i] >> (sh - 4);  // the 2-bit field to bits 4, 5
            v[i] = (hs & 0x30303030u) | lo;
        }
        return (long)(((uint64_t)v[1] << 32) | v[0]);
    }
    // The factors of a block, decoded by the wave once: lane (c, q) takes row c's sub-blocks 2q and 2q + 1, both
    // halves of each -- scales[4q .. 4q + 3], table slots 4q .. 4q + 3 (slot = 2 * sub-block + half).
    template <int U>
    static __device__ __forceinline__ void block_factors(const uint8_t *blk, uint32_t q, float (&f)[4]) {
        const uint32_t sc = strip_get4<2 * U>(blk + 192 + 4 * q);
        const float d = h2f(reinterpret_cast<const StripR2 *>(blk + 208)->v);
#pragma unroll
        for (int b = 0; b < 4; b++) f[b] = d * (float)(int)(int8_t)((sc >> (8 * b)) & 0xFF);  // reference/q6_k.rs:62, exact
    }
};

// LDS bytes per (sub-block, token tile): int8 operands, fp32 scales, and fp32 P (one factor per sub-block) or the
// MFMA addends of the two halves (two factors; with a zero-point term, P of each half as well)
template <class F>
constexpr uint32_t skinny_act_bytes() {
    return 512 + 64 + (Skinny<F>::KSPLIT == 2 ? 128 : 64) + (Skinny<F>::KSPLIT == 2 && Skinny<F>::HAS_MIN ? 128 : 0);
}
constexpr uint32_t SKINNY_FAC_STRIDE = 17;  // floats per weight row in a wave's factor tables (16 + pad)
// LDS bytes of a wave: the strip of its rows' bytes of a step, and the factor tables (one factor per sub-block: of
// the step's 16 sub-blocks, and a second table where the format has a zero-point term; two factors: of one block's)
template <class F, int NT>
constexpr uint32_t skinny_wave_lds() {
    return NT * 16 * (Skinny<F>::ROW_STRIDE + (Skinny<F>::TABLE ? SKINNY_FAC_STRIDE * 4 * (Skinny<F>::HAS_MIN ? 2 : 1) : 0));
}

typedef float v4f32 __attribute__((ext_vector_type(4)));
struct __attribute__((packed, aligned(4))) StripA4 { u32x4 v; };

// Work group = WAVES waves, each with its own NT x 16 weight rows; all of them the same token tiles (at most TT of
// 16 tokens).  k is walked in chunks of `per` super-blocks (even): the work group stages the chunk's token bytes,
// every wave runs its rows over the chunk, accumulators staying in registers; the weight prefetch runs on across
// the chunk boundary.  blockIdx.x = row group, blockIdx.y = expert (grouped form), blockIdx.z = token pass.
// One matrix (no experts) with too few row groups to fill the chip: blockIdx.y = which sb_per_split super-blocks of
// k the work group walks; it stores its sums to partial[blockIdx.y][token][row] and gemm_skinny_reduce adds the
// splits in index order.
// LDS: [A operands | fp32 token scales | P] of a chunk, then per wave [weight strip | dsc table | zero-point table].
// Waves per SIMD the shape is meant to run at: two work groups on a compute unit where their LDS allows it.
template <class F, int NT, int WAVES, int TT, int PER>
constexpr int skinny_waves_per_simd() {
    constexpr size_t lds = (size_t)PER * 8 * TT * skinny_act_bytes<F>() + (size_t)WAVES * skinny_wave_lds<F, NT>();
    return lds <= 80 * 1024 ? WAVES / 2 : WAVES / 4;
}

// The work of one work group on the token rows tokb .. tok_end - 1 (at most 16 * TT of them) of its group.
// SPREAD_LOG (two token tiles only): the second tile's rows sit in every 2^SPREAD_LOG-th of its 16 slots.  A lane's four
// results of an MFMA are the slots 4q .. 4q + 3, so with up to 4 (8) rows in the second tile only one (two) of them
// is a token and the two fmas of each of the others are not compiled in.
template <class F, int NT, int WAVES, int TT, int PER, bool DUMP, int SPREAD_LOG = 0>
__device__ __forceinline__ void gemm_skinny_body(
    const uint8_t *__restrict__ W, const uint8_t *__restrict__ A, float *__restrict__ out, int32_t *__restrict__ sums,
    uint32_t m, uint32_t n, uint32_t k, int accumulate, const float *__restrict__ bias, const int32_t *__restrict__ offsets, size_t w_stride,
    float *__restrict__ partial, uint32_t sb_per_split, const uint32_t tokb, const uint32_t tok_end, const uint32_t rg,
    const uint32_t gy, const uint32_t ks) {
    using S = Skinny<F>;
    constexpr float MAGIC = 12582912.0f;  // 1.5 * 2^23: as_float(0x4B400000 + i) == MAGIC + i for |i| < 2^22
    constexpr int KS = S::KSPLIT;  // MFMAs (and scale factors) per sub-block
    // a row's bytes of a step as 16-byte pieces: FULL whole ones from the start, and where the step's length is not
    // a multiple of 16 one more that ends with the step (overlapping the last whole one).  Four lanes share a row:
    // a load instruction takes 64 consecutive bytes of each of 16 rows, the next one the next 64, so that a lane's
    // pieces sit at fixed distances from its first (one address register, one LDS offset register); only the last
    // instruction of a row, where the pieces run out, has offsets of its own.
    constexpr uint32_t RS = S::ROW_STRIDE, SEG = 2 * S::BLOCK, FULL = SEG / 16, TAIL = SEG % 16 ? 1 : 0;
    constexpr uint32_t PPR = FULL + TAIL, ITR = (PPR + 3) / 4, NL = NT * ITR;
    constexpr uint32_t THREADS = 64 * WAVES, FS = SKINNY_FAC_STRIDE;
    constexpr uint32_t WAVE_LDS = skinny_wave_lds<F, NT>();
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    const uint32_t lane = threadIdx.x & 63, c = lane & 15, q = lane >> 4;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    // super-blocks [sb_lo, n_super) of this work group (all of k, or its split)
    const uint32_t sb_lo = partial ? ks * sb_per_split : 0;
    const uint32_t n_super = partial ? min(k / 256, sb_lo + sb_per_split) : k / 256;
    const bool odd_super = (n_super & 1) != 0;  // (sb_lo is even: only the end of k can leave half a step)
    constexpr uint32_t per = PER, nblk_max = PER * 8;  // sub-blocks (Q8_0 blocks per token) of a full chunk
    uint8_t *const ldsA = lds;
    float *const ldsD = reinterpret_cast<float *>(ldsA + (size_t)nblk_max * TT * 512);
    float *const ldsP = ldsD + (size_t)nblk_max * TT * 16;       // one factor per sub-block: P
    int *const ldsC = reinterpret_cast<int *>(ldsP);             // two: the MFMA addends, [block][tile][half][16 tokens]
    float *const ldsP2 = ldsP + (size_t)nblk_max * TT * 16 * KS;  // two factors and a zero-point term: P per half
    uint8_t *const strip = reinterpret_cast<uint8_t *>(ldsP2 + (KS == 2 && S::HAS_MIN ? (size_t)nblk_max * TT * 32 : 0)) + wave * WAVE_LDS;
    float *const dscT = reinterpret_cast<float *>(strip + NT * 16 * RS);
    float *const minT = dscT + NT * 16 * FS;

    // ---- a chunk's tokens: their Q8_0 blocks (34 bytes: f16 scale, 32 int8) from the caller's rows into registers
    // (requested a chunk ahead, in flight while the last chunk is computed), from there into LDS in operand order,
    // with what gemm_prep_acts would have made of them: the bytes of each 8 in the format's order, the scale as
    // fp32, P = d * sum(q) (exact integer sum, one rounding).  Thread (cc, qq) of a 64-thread unit takes bytes
    // 8 qq .. 8 qq + 7 of token cc's block; token rows past the group's end read as zeros. ----
    constexpr uint32_t KA = (nblk_max * TT * 64 + THREADS - 1) / THREADS;
    const size_t arow = (size_t)(k / 32) * Q8_BLOCK_BYTES;
    static_assert(SPREAD_LOG == 0 || TT == 2, "spread slots: the second token tile");
    constexpr uint32_t DEAD_SLOTS = (1u << SPREAD_LOG) - 1;  // the second tile's slot holds a token where slot & DEAD_SLOTS == 0
    // token row of slot `slot` of tile t, or tok_end (none)
    auto token_of = [&](uint32_t t, uint32_t slot) {
        if (SPREAD_LOG != 0 && t == 1) return (slot & DEAD_SLOTS) ? tok_end : tokb + 16 + (slot >> SPREAD_LOG);
        return tokb + 16 * t + slot;
    };
    u32x2 tokA[KA];
    uint32_t tokD[KA];
    auto load_tokens = [&](uint32_t sb0, uint32_t nblk) {
        const uint32_t total = nblk * TT * 64;
#pragma unroll
        for (uint32_t i = 0; i < KA; i++) {
            const uint32_t idx = threadIdx.x + i * THREADS;
            const uint32_t l = idx & 63, t = (idx >> 6) % TT, b = (idx >> 6) / TT;
            const uint32_t cc = l >> 2, qq = l & 3, tok = token_of(t, cc);
            tokA[i] = u32x2{0, 0};
            tokD[i] = 0;
            // an odd number of super-blocks: the last step's strip holds the last two super-blocks, the one before the
            // last (done by the step before) in its first half -- that half meets zeros, the second the last one's tokens
            uint32_t sbi = sb0 + (b >> 3);
            const bool dead = odd_super && sbi == n_super - 1;
            if (odd_super && sbi == n_super) sbi = n_super - 1;
            if (idx < total && tok < tok_end && !dead) {
                const uint8_t *blk = A + (size_t)tok * arow + (size_t)(sbi * 8 + (b & 7)) * Q8_BLOCK_BYTES;
                tokA[i] = ld8(blk + 2 + 8 * qq);
                tokD[i] = ld2(blk);
            }
        }
    };
    auto store_tokens = [&](uint32_t nblk) {
        const uint32_t total = nblk * TT * 64;
#pragma unroll
        for (uint32_t i = 0; i < KA; i++) {
            const uint32_t idx = threadIdx.x + i * THREADS;
            if (idx >= total) continue;  // whole waves: total and THREADS are multiples of 64
            const uint32_t l = idx & 63, cc = l >> 2, qq = l & 3;
            u32x2 v = tokA[i];
            const float d = h2f(tokD[i]);
            if constexpr (S::HAS_MIN && KS == 1) {
                int sum = sdot4(v[0], 0x01010101u, sdot4(v[1], 0x01010101u, 0));
                sum += xor1_i(sum);  // the four threads of a block
                sum += xor2_i(sum);
                if (qq == 0) ldsP[(idx >> 6) * 16 + cc] = d * (float)sum;
            }
            if constexpr (S::HAS_MIN && KS == 2) {  // a zero-point factor per 16 weights: P of each half
                int sum = sdot4(v[0], 0x01010101u, sdot4(v[1], 0x01010101u, 0));
                sum += xor1_i(sum);
                if ((qq & 1) == 0) ldsP2[((idx >> 6) * 2 + (qq >> 1)) * 16 + cc] = d * (float)sum;
            }
            if constexpr (KS == 2) {
                // per half of the block (threads 0, 1 and 2, 3): the addend that turns sum(q a) into sum((q - OFFSET) a),
                // on top of the 1.5 * 2^23 every result carries
                int sum = sdot4(v[0], 0x01010101u, sdot4(v[1], 0x01010101u, 0));
                sum += xor1_i(sum);
                if ((qq & 1) == 0) ldsC[((idx >> 6) * 2 + (qq >> 1)) * 16 + cc] = 0x4B400000 - S::OFFSET * sum;
            }
            if (S::ACT_PERM == 1) {  // even bytes, then odd bytes
                const uint32_t x0 = v[0], x1 = v[1];
                v[0] = __builtin_amdgcn_perm(x1, x0, 0x06040200u);
                v[1] = __builtin_amdgcn_perm(x1, x0, 0x07050301u);
            }
            if constexpr (S::ACT_PERM == 2) {
                // weights j and j + 16 share a byte: k-slot q holds token bytes 4q .. 4q + 3, then 16 + 4q .. 16 + 4q + 3
#pragma unroll
                for (uint32_t i = 0; i < 2; i++)
                    *reinterpret_cast<uint32_t *>(ldsA + ((size_t)(idx >> 6) * 64 + (2 * (qq & 1) + i) * 16 + cc) * 8 + 4 * (qq >> 1)) = v[i];
            } else {
                *reinterpret_cast<u32x2 *>(ldsA + ((size_t)(idx >> 6) * 64 + qq * 16 + cc) * 8) = v;
            }
            if (qq == 0) ldsD[(idx >> 6) * 16 + cc] = d;
        }
    };

    const uint32_t steps = (n_super + 1) / 2;
    const uint32_t rbase = (rg * WAVES + wave) * (16 * NT);
    const bool active = rbase < n;  // a wave past the last row still stages tokens and meets the barriers
    const uint8_t *We = W + (offsets ? (size_t)gy * w_stride : 0);
    const size_t row_bytes = (size_t)(k / 256) * S::BLOCK;
    // the lane's pieces of a step: where they come from (less the step's offset) and where they go
    const uint32_t lrow = lane >> 2, sub = lane & 3;
    const uint8_t *src[NT];
    uint32_t dst[NT];
#pragma unroll
    for (uint32_t j = 0; j < NT; j++) {
        src[j] = We + (size_t)min(rbase + 16 * j + lrow, n - 1) * row_bytes + 16 * sub;
        dst[j] = (16 * j + lrow) * RS + 16 * sub;
    }
    // the row's last instruction: piece sub + 4 (ITR - 1), or the row's last piece where that is past it (loaded by
    // several lanes then, and stored to the same place with the same value)
    const uint32_t last_piece = min(sub + 4 * (ITR - 1), PPR - 1);
    const uint32_t last_at = ((TAIL && last_piece == PPR - 1) ? SEG - 16 : 16 * last_piece) - 16 * sub;
    auto load_step = [&](u32x4 (&stage)[NL], uint32_t st) {
#pragma unroll
        for (uint32_t j = 0; j < NT; j++) {
            const uint8_t *sp = src[j] + (odd_super && st == steps - 1 ? (size_t)(n_super - 2) * S::BLOCK : (size_t)st * SEG);
#pragma unroll
            for (uint32_t i = 0; i < ITR; i++) stage[j * ITR + i] = ld16(sp + (i + 1 < ITR ? 64 * i : last_at));
        }
    };
    const uint32_t tiles_here = min((uint32_t)TT, (tok_end - tokb + 15) / 16);
    v4f32 acc[TT][NT];
#pragma unroll
    for (int t = 0; t < TT; t++)
#pragma unroll
        for (int j = 0; j < NT; j++) acc[t][j] = v4f32{0.0f, 0.0f, 0.0f, 0.0f};

    // the MFMA's addend, 1.5 * 2^23 in every element: made opaque so that it stays in one register quad for the whole
    // walk (as a plain constant the compiler rebuilds three of the four registers before every MFMA)
    v4i32 magic;
    asm volatile("v_mov_b32 %0, 0x4b400000\n\tv_mov_b32 %1, 0x4b400000\n\tv_mov_b32 %2, 0x4b400000\n\tv_mov_b32 %3, 0x4b400000"
                 : "=v"(magic[0]), "=v"(magic[1]), "=v"(magic[2]), "=v"(magic[3]));
    const uint64_t half_mask = q < 2 ? ~0ull : 0ull;
    u32x4 stage[NL];
    load_step(stage, sb_lo / 2);
    // (token blocks are staged by whole steps: an odd last super-block brings a dead one along)
    auto chunk_blocks = [&](uint32_t from) { return ((min(per, n_super - from) + 1) & ~1u) * 8; };
    load_tokens(sb_lo, chunk_blocks(sb_lo));
    for (uint32_t sb0 = sb_lo; sb0 < n_super; sb0 += per) {
    const uint32_t nsbc = (min(per, n_super - sb0) + 1) & ~1u;
    __syncthreads();  // every wave is done with the last chunk's tokens
    store_tokens(nsbc * 8);
    __syncthreads();
    if (sb0 + per < n_super) load_tokens(sb0 + per, chunk_blocks(sb0 + per));
    // The chunk's steps.  One token tile: no branch inside a step, so the LDS reads, the MFMAs and the fmas of
    // different sub-blocks interleave.  Two: each tile's work sits behind a branch on the group's tile count --
    // measured faster than the branch-free form, which needs more registers than two work groups per
    // compute unit leave (14336 x 4096, 8 experts, mean 12 rows: 88 us against 101).
    {
    constexpr int TN = TT;
    if (active)
    for (uint32_t st = sb0 / 2; st < (sb0 + nsbc) / 2; st++) {
        // the step's bytes to the strip (pieces past the end, on the last load: the last piece again, same value)
#pragma unroll
        for (uint32_t j = 0; j < NT; j++)
#pragma unroll
            for (uint32_t i = 0; i < ITR; i++) {
                if (i + 1 < ITR)
                    *reinterpret_cast<u32x4 *>(strip + dst[j] + 64 * i) = stage[j * ITR + i];
                else if (TAIL)  // the rows' last pieces among them: on dword boundaries only
                    reinterpret_cast<StripA4 *>(strip + dst[j] + last_at)->v = stage[j * ITR + i];
                else
                    *reinterpret_cast<u32x4 *>(strip + dst[j] + last_at) = stage[j * ITR + i];
            }
        if (st + 1 < steps) load_step(stage, st + 1);
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        // scale factors of the step, decoded once: lane (c, q) takes row c, super-block q / 2, sub-blocks
        // 4 (q % 2) .. + 3, for each tile (two factors per sub-block: per block, below)
        if constexpr (KS == 1 && S::TABLE)
#pragma unroll
        for (int j = 0; j < NT; j++) {
            typename S::Raw hd;
            S::read_hdr(hd, strip + (16 * j + c) * RS + (q >> 1) * S::BLOCK, q & 1);
#pragma unroll
            for (int i = 0; i < 4; i++) {
                float dsc, qneg;
                S::factors(hd, q & 1, i, dsc, qneg);
                dscT[(16 * j + c) * FS + 4 * q + i] = dsc;
                if (S::HAS_MIN) minT[(16 * j + c) * FS + 4 * q + i] = qneg;
            }
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
        for (int u = 0; u < 2; u++) {
            typename S::Raw raw[NT];
#pragma unroll
            for (int j = 0; j < NT; j++) {  // (u is a constant once the loop is unrolled)
                const uint8_t *blk = strip + (16 * j + c) * RS + u * S::BLOCK;
                if (u == 0) S::template read<0>(raw[j], blk, q);
                else S::template read<1>(raw[j], blk, q);
            }
            const uint32_t b0 = (st * 2 + u - sb0) * 8;
            if constexpr (KS == 2) {
                // the block's factors (the table holds one block's: the last block's readers are done)
                __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
                __builtin_amdgcn_wave_barrier();
#pragma unroll
                for (int j = 0; j < NT; j++) {
                    float f[4];
                    const uint8_t *blk = strip + (16 * j + c) * RS + u * S::BLOCK;
                    if constexpr (S::HAS_MIN) {
                        float mn[4];
                        if (u == 0) S::template block_factors<0>(blk, q, f, mn);
                        else S::template block_factors<1>(blk, q, f, mn);
#pragma unroll
                        for (int b = 0; b < 4; b++) minT[(16 * j + c) * FS + 4 * q + b] = mn[b];
                    } else {
                        if (u == 0) S::template block_factors<0>(blk, q, f);
                        else S::template block_factors<1>(blk, q, f);
                    }
#pragma unroll
                    for (int b = 0; b < 4; b++) dscT[(16 * j + c) * FS + 4 * q + b] = f[b];
                }
                __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
                __builtin_amdgcn_wave_barrier();
                __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
            }
            if constexpr (S::HAS_MIN && KS == 2) {
                // zero-point term, a factor per 16 weights: per four halves (slot = 2 * sub-block + half) one
                // 16 x 16 x 4 fp32 product of P (tokens x halves) and the rows' factors of the block
#pragma unroll
                for (int g = 0; g < 4; g++)
#pragma unroll
                    for (int t = 0; t < TN; t++)
                        if (TT == 1 || t < (int)tiles_here) {
                            const float pa = ldsP2[(((b0 + 2 * g + (q >> 1)) * TT + t) * 2 + (q & 1)) * 16 + c];
#pragma unroll
                            for (int j = 0; j < NT; j++) {
                                const float zb = minT[(16 * j + c) * FS + 4 * g + q];
                                acc[t][j] = __builtin_amdgcn_mfma_f32_16x16x4f32(pa, zb, acc[t][j], 0, 0, 0);
                            }
                        }
            }
            if constexpr (S::HAS_MIN && KS == 1) {
                // zero-point term: per four sub-blocks one 16 x 16 x 4 fp32 product of P (tokens x sub-blocks) and the
                // rows' factors, straight into the accumulators
#pragma unroll
                for (int hf = 0; hf < 2; hf++)
#pragma unroll
                    for (int t = 0; t < TN; t++)
                        if (TT == 1 || t < (int)tiles_here) {
                            const float pa = ldsP[((b0 + 4 * hf + q) * TT + t) * 16 + c];
#pragma unroll
                            for (int j = 0; j < NT; j++) {
                                const float zb = minT[(16 * j + c) * FS + u * 8 + 4 * hf + q];
                                acc[t][j] = __builtin_amdgcn_mfma_f32_16x16x4f32(pa, zb, acc[t][j], 0, 0, 0);
                            }
                        }
            }
#pragma unroll
            for (int s = 0; s < 8; s++) {
                float dsc[NT][KS], corr[NT][KS];
                long bop[NT][KS];
#pragma unroll
                for (int j = 0; j < NT; j++) {
                    const long op = S::operand(raw[j], s);
#pragma unroll
                    for (int is = 0; is < KS; is++) {
                        if constexpr (S::TABLE) dsc[j][is] = dscT[(16 * j + c) * FS + (KS == 2 ? 2 * s + is : u * 8 + s)];
                        else dsc[j][is] = S::scale(raw[j], s);
                        corr[j][is] = -(MAGIC * dsc[j][is]);
                        // two factors: k-values 0..15 come from the lanes q = 0, 1, the others supply zeros; and so on
                        bop[j][is] = KS == 2 ? (long)((uint64_t)op & (is == 0 ? half_mask : ~half_mask)) : op;
                    }
                }
#pragma unroll
                for (int t = 0; t < TN; t++) {
                    if (TT == 1 || t < (int)tiles_here) {
                        const uint32_t e = (b0 + s) * TT + t;
                        const u32x2 av = *reinterpret_cast<const u32x2 *>(ldsA + ((size_t)e * 64 + lane) * 8);
                        const long a = (long)(((uint64_t)av[1] << 32) | av[0]);
                        const v4f32 da = *reinterpret_cast<const v4f32 *>(ldsD + (size_t)e * 16 + 4 * q);
#pragma unroll
                        for (int is = 0; is < KS; is++) {
                            v4i32 addend = magic;
                            if constexpr (KS == 2) addend = *reinterpret_cast<const v4i32 *>(ldsC + ((size_t)e * 2 + is) * 16 + 4 * q);
#pragma unroll
                            for (int j = 0; j < NT; j++) {
                                const v4i32 r = __builtin_amdgcn_mfma_i32_16x16x32_i8(a, bop[j][is], addend, 0, 0, 0);
#pragma unroll
                                for (int v = 0; v < 4; v++) {
                                    if (SPREAD_LOG != 0 && t == 1 && (v & DEAD_SLOTS)) continue;  // a slot without a token
                                    const int ri = r[v];
                                    const float tt = fmaf(__builtin_bit_cast(float, ri), dsc[j][is], corr[j][is]);  // fl(dsc * isum)
                                    acc[t][j][v] = fmaf(tt, da[v], acc[t][j][v]);
                                    if (DUMP) {  // the integer sum of (token, weight row, sub-block or half of one)
                                        const uint32_t tok = token_of(t, 4 * q + v), row = rbase + 16 * j + c;
                                        // (the odd last step: its first half is the dead one, its second the last super-block)
                                        const bool last_odd = odd_super && st == steps - 1;
                                        const uint32_t sbi = last_odd ? n_super - 1 : st * 2 + u;
                                        if (tok < tok_end && row < n && !(last_odd && u == 0))
                                            sums[((size_t)tok * n + row) * (k / 32 * KS) + (sbi * 8 + s) * KS + is] =
                                                ri - 0x4B400000;
                                    }
                                }
                            }
                        }
                    }
                }
            }
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
    }
    }
    }
#pragma unroll
    for (int t = 0; t < TT; t++)
#pragma unroll
        for (int j = 0; j < NT; j++) {
            const uint32_t row = rbase + 16 * j + c;
#pragma unroll
            for (int v = 0; v < 4; v++) {
                const uint32_t tok = token_of(t, 4 * q + v);
                if (row < n && tok < tok_end && t < (int)tiles_here) {
                    const float y = acc[t][j][v];
                    if (partial) {
                        partial[((size_t)ks * m + tok) * n + row] = y;
                    } else {
                        float *o = out + (size_t)tok * n + row;
                        *o = accumulate ? *o + y : bias ? y + bias[row] : y;
                    }
                }
            }
        }
}

// The kernel: finds the work group's token rows and runs the body.  A launch shaped for two token tiles runs the
// one-tile body (same LDS bytes: twice the chunk length) for a group that has rows in the first tile only -- the
// branch-free step instead of the two-tile step's branches, for what is most of the groups when the mean is 16 rows.
template <class F, int NT, int WAVES, int TT, int PER, bool DUMP>
__global__ __launch_bounds__(64 * WAVES)
__attribute__((amdgpu_waves_per_eu(skinny_waves_per_simd<F, NT, WAVES, TT, PER>(), skinny_waves_per_simd<F, NT, WAVES, TT, PER>())))
void gemm_skinny_kernel(
    const uint8_t *__restrict__ W, const uint8_t *__restrict__ A, float *__restrict__ out, int32_t *__restrict__ sums,
    uint32_t m, uint32_t n, uint32_t k, int accumulate, const float *__restrict__ bias, const int32_t *__restrict__ offsets, size_t w_stride,
    float *__restrict__ partial, uint32_t sb_per_split, uint32_t grouped_splits) {
    // row group; expert (grouped form); split of k: blockIdx.y is the expert, or the split (one matrix), or, in the
    // grouped form with k split, expert * grouped_splits + split
    const uint32_t rg = blockIdx.x;
    uint32_t gy = !offsets ? 0 : partial ? blockIdx.y / grouped_splits : blockIdx.y;
    const uint32_t ks = !partial ? 0 : offsets ? blockIdx.y % grouped_splits : blockIdx.y;
    if constexpr (TT == 2) {
        // Groups of two token tiles take longer than groups of one: hand the experts out largest group first
        // (ties by index), so that the long work groups start in the first round and the short ones fill the end.
        // Lane e ranks expert e; the work group takes the expert whose rank is its place in the grid.
        const uint32_t n_e = offsets ? gridDim.y / (partial ? grouped_splits : 1u) : 0u;
        if (n_e > 1 && n_e <= 64) {
            const uint32_t lane = threadIdx.x & 63, e = min(lane, n_e - 1);
            const int size_e = offsets[e + 1] - offsets[e];
            uint32_t rank = 0;
            for (uint32_t o = 0; o < n_e; o++) {
                const int so = __builtin_amdgcn_readlane(size_e, (int)o);
                rank += (so > size_e || (so == size_e && o < e)) ? 1u : 0u;
            }
            const unsigned long long hit = __ballot(lane < n_e && rank == gy);
            gy = (uint32_t)__builtin_amdgcn_readfirstlane((int)(__ffsll((long long)hit) - 1));
        }
    }
    uint32_t tok0 = 0, tok_end = m;
    if (offsets) {
        tok0 = (uint32_t)offsets[gy];
        tok_end = (uint32_t)offsets[gy + 1];
    }
    // blockIdx.z = which 16 * TT token rows of the group: the launch is shaped for the usual group, a larger one
    // takes further work groups per row group (each its own pass over the weights); the rest exit here.
    // (One token tile: the second pass is dispatched before the first, so that the few work groups of the groups
    // that overflow run beside the first pass instead of after it; further passes, nearly always empty, come last.
    // Two tiles: overflow is rare, and a layer of work groups that only exit would delay the start.  Walking the
    // passes in a loop inside the work group instead of by layers of the grid was measured 7-9 % slower on every
    // shape: the compiler allocates the looped body worse.)
    const uint32_t pass = (TT == 1 && gridDim.z > 1 && blockIdx.z < 2) ? 1 - blockIdx.z : blockIdx.z;
    const uint32_t tokb = tok0 + pass * (16 * TT);
    if (tokb >= tok_end) return;  // the whole work group
    if constexpr (TT == 2) {
        if (tok_end - tokb <= 16) {
            gemm_skinny_body<F, NT, WAVES, 1, 2 * PER, DUMP>(W, A, out, sums, m, n, k, accumulate, bias, offsets, w_stride,
                                                            partial, sb_per_split, tokb, tok_end, rg, gy, ks);
            return;
        }
    }
    if constexpr (TT == 2 && !DUMP) {
        // a second tile of up to 4 (8) rows: the body that spreads them over the slots (same sums, same order)
        if (tok_end - tokb <= 20) {
            gemm_skinny_body<F, NT, WAVES, TT, PER, DUMP, 2>(W, A, out, sums, m, n, k, accumulate, bias, offsets, w_stride,
                                                             partial, sb_per_split, tokb, tok_end, rg, gy, ks);
            return;
        }
        if (tok_end - tokb <= 24) {
            gemm_skinny_body<F, NT, WAVES, TT, PER, DUMP, 1>(W, A, out, sums, m, n, k, accumulate, bias, offsets, w_stride,
                                                             partial, sb_per_split, tokb, tok_end, rg, gy, ks);
            return;
        }
    }
    gemm_skinny_body<F, NT, WAVES, TT, PER, DUMP>(W, A, out, sums, m, n, k, accumulate, bias, offsets, w_stride, partial,
                                                  sb_per_split, tokb, tok_end, rg, gy, ks);
}

// out[i] (+)= partial[0][i] + partial[1][i] + ... in that order, i over m x n; bias[row] instead of the old value
// when the call overwrites.  V = 4: four consecutive elements per thread (n a multiple of 4, buffers 16-byte aligned).
template <int V>
static __global__ __launch_bounds__(256) void gemm_skinny_reduce(const float *__restrict__ partial, float *__restrict__ out,
                                                                const float *__restrict__ bias, size_t total, uint32_t n,
                                                                uint32_t splits, int accumulate) {
    const size_t i = ((size_t)blockIdx.x * 256 + threadIdx.x) * V;
    if (i >= total) return;
    float y[V];
    if (V == 4) {
        const v4f32 p0 = *reinterpret_cast<const v4f32 *>(partial + i);
        for (int v = 0; v < V; v++) y[v] = p0[v];
        for (uint32_t s = 1; s < splits; s++) {
            const v4f32 ps = *reinterpret_cast<const v4f32 *>(partial + (size_t)s * total + i);
            for (int v = 0; v < V; v++) y[v] += ps[v];
        }
    } else {
        y[0] = partial[i];
        for (uint32_t s = 1; s < splits; s++) y[0] += partial[(size_t)s * total + i];
    }
    for (int v = 0; v < V; v++) out[i + v] = accumulate ? out[i + v] + y[v] : bias ? y[v] + bias[(i + v) % n] : y[v];
}

// Super-blocks per split of k for one matrix of n rows (0: no split): enough splits for about 1.75 work groups of 128
// rows per compute unit of a 256-CU part, at least two steps (four super-blocks) each, at most 16.  A function of the
// shape alone, so that the workspace size is.
static inline uint32_t skinny_sb_per_split(uint32_t n, uint32_t k) {
    const uint32_t n_super = k / 256, groups = (n + 127) / 128;
    // Small matrices: with rows of 4096 columns and more the split still beats the tile kernel's few, long work groups
    // (16 rows, us: 2048 x 8192 12.1 against 18.3, 1536 x 8960 13.4 against 20.0, 512 x 8192 10.8 against 17.2, 4096 x
    // 4096 10.9 against 12.6, 1024 x 4096 9.5 against 11.7); with shorter rows it is a tie (2048 x 2048 9.1 against
    // 8.9), and below 2^22 weights the two launches cost more than they save
    const uint64_t weights = (uint64_t)n * k;
    if (k % 256 != 0 || groups >= 448 || weights < (1ull << 22) || (k < 4096 && weights < (1ull << 25))) return 0;
    uint32_t splits = (448 + groups - 1) / groups;
    if (splits > 16) splits = 16;
    if (splits > n_super / 4) splits = n_super / 4;
    if (splits < 2) return 0;
    return ((n_super + splits - 1) / splits + 1) & ~1u;
}
static inline uint32_t skinny_splits(uint32_t n, uint32_t k) {
    const uint32_t per = skinny_sb_per_split(n, k);
    return per ? (k / 256 + per - 1) / per : 1;
}

// Grouped form: an expert's k is split in two where its matrix has too few row groups to fill the chip by experts
// alone (at most this many rows per expert; the workspace size follows the same bound).
constexpr uint32_t SKINNY_GROUPED_SPLITS = 2, SKINNY_GROUPED_SPLIT_MAX_N = 8192;

template <class F, int NT, int WAVES, int TT, int PER, bool DUMP = false>
static hipError_t launch_skinny_shape(const GemmArgs &a, const TilePlan &p, hipStream_t stream, bool split_k = false) {
    const size_t strips = (size_t)WAVES * skinny_wave_lds<F, NT>();
    auto kern = &gemm_skinny_kernel<F, NT, WAVES, TT, PER, DUMP>;
    const size_t lds = (size_t)PER * 8 * TT * skinny_act_bytes<F>() + strips;
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                                       (int)lds);
    if (e != hipSuccess) return e;
    // token passes: as many as the largest group can need (max_rows is the caller's bound, all rows if unknown)
    const uint32_t group_rows = a.offsets ? a.max_rows : a.m;
    const uint32_t splits = !split_k ? 1 : a.offsets ? SKINNY_GROUPED_SPLITS : skinny_splits(a.n, a.k);
    float *const partial = splits > 1 ? p.partial : nullptr;
    if (splits > 1 && !partial) return hipErrorNotSupported;
    // super-blocks per split: the grouped form halves k (a multiple of 1024: whole steps in both halves)
    const uint32_t sb_per_split = a.offsets ? a.k / 256 / SKINNY_GROUPED_SPLITS : skinny_sb_per_split(a.n, a.k);
    if (splits > 1 && a.offsets && a.k % (512 * SKINNY_GROUPED_SPLITS) != 0) return hipErrorNotSupported;
    const uint32_t row_groups = (a.n + 16 * NT * WAVES - 1) / (16 * NT * WAVES);
    const dim3 grid(row_groups, a.offsets ? a.n_experts * splits : splits, (group_rows + 16 * TT - 1) / (16 * TT));
    if (grid.z > 65535 || grid.y > 65535) return hipErrorNotSupported;
    note_launch("gemm_skinny_kernel", F::TYPE, NT, WAVES, TT, PER, grid.x, grid.y * grid.z, 64 * WAVES);
    hipLaunchKernelGGL(kern, grid, dim3(64 * WAVES), lds, stream, a.W, a.A, a.out, a.sums, a.m, a.n, a.k,
                       a.accumulate, a.bias, a.offsets, a.w_stride, partial, sb_per_split, splits);
    e = hipGetLastError();
    if (e != hipSuccess || !partial) return e;
    if (a.defer_reduce && !a.accumulate && !a.bias) {  // the caller adds the splits' sums (in index order, as below)
        a.defer_reduce->partial = partial;
        a.defer_reduce->splits = splits;
        return hipSuccess;
    }
    const size_t total = (size_t)a.m * a.n;
    if (a.n % 4 == 0 && (reinterpret_cast<uintptr_t>(a.out) & 15) == 0)
        hipLaunchKernelGGL(gemm_skinny_reduce<4>, dim3((unsigned)((total / 4 + 255) / 256)), dim3(256), 0, stream, partial,
                           a.out, a.bias, total, a.n, splits, a.accumulate);
    else
        hipLaunchKernelGGL(gemm_skinny_reduce<1>, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, stream, partial, a.out,
                           a.bias, total, a.n, splits, a.accumulate);
    return hipGetLastError();
}

// Which launch shape serves a call: 0 = none (not this format / shape, or one the tile kernel serves better).  rows =
// the token rows per group the launch is shaped for; has_partial: the workspace has room for split-k sums.
// variant 0: the measured choice; 200..205: a fixed shape (tuning, tests).
// Measured on MI355X, 8 experts of Mixtral's shapes (IQ4_XS; Q4_K alike), cold weights, against the tile kernel:
//  * up to 16 rows per expert: 14336 x 4096 84 us against 106, 4096 x 14336 90 against 107;
//  * 17..32 rows: two token tiles double the arithmetic per weight byte.  With a mean of 12 rows (most experts still
//    one tile) 14336 x 4096 takes 88 us against 102; with a mean of 16 the kernel alone is 93 us against 103, and
//    the tile kernel's token re-layout launch (5 us) is not needed: the layer of 64 tokens 311-317 us against
//    340-343; 4096 x 14336 (one work group per compute unit, the longer per-step chain uncovered) 126 against 106,
//    and with each expert's k in two halves (twice the work groups, a reduction launch) 90 + 5 against 103 + 5: the
//    layer 293-303 us;
//  * one matrix, no experts, up to 16 token rows: too few row groups as it is (14336 x 4096: 24 us against 19);
//    with k split over work groups and the splits added by a second launch (call totals, with the token re-layout):
//    14336 x 4096 18.0 us against 19.6, 4096 x 14336 21.4 against 29.5, 28672 x 8192 40 against 49; 4096 x 4096
//    14.4 against 12.3 (not taken below 2^25 weights); 17..32 rows 24.6 against 19.7 (not taken).  From 512 row
//    groups on no split is needed (57344 x 4096, 16 rows: 44 us against 56).
enum SkinnyShape { SK_NONE = 0, SK_1_4, SK_1_8, SK_2_2, SK_1_4_SPLIT, SK_1_16, SK_2_8, SK_W4_1_8, SK_W4_2_4, SK_2_4, SK_2_2_SPLIT };

// Expert groups of up to this many rows in the mean stay with the kernel's two-tile shapes (larger groups take further
// passes over their expert's weights).  20 where the tile kernel is the alternative at its best (Q4_K, IQ4_XS: 8
// experts of 14336 x 4096 with 13..28 rows 92-101 us against 105 + 5); the formats of 32-weight blocks, whose tile
// kernel is bound by its many small loads, keep the few-token kernel up to 48 (the Mixtral-shaped layer at 96 / 128 /
// 192 tokens, us: Q4_1 348 / 436 / 625 against 527 / 671 / 712 on the tile kernel, Q4_0 348 / 440 / 630 against 486 /
// 619 / 663, IQ4_NL 331 / 438 / 627 against 490 / 628 / 648; at 256 tokens, a mean of 64, the tile kernel is level).
template <class F>
constexpr uint32_t skinny_grouped_mean_limit() {
    return tile_ragged_k<F>::value ? 48 : 20;
}

template <class F>
static int skinny_shape(const GemmArgs &a, bool has_partial, uint32_t rows, int variant) {
    if constexpr (Skinny<F>::OK) {
        constexpr size_t MEAN_LIMIT = skinny_grouped_mean_limit<F>();
        // whole steps of two super-blocks
        // (expert groups of a mean of up to 20 rows: the launch may be shaped for more than 32 -- twice the mean --
        // and the groups beyond 32 rows take further passes)
        if (a.k % 256 != 0 || a.k < 512 || (rows > 32 && !(a.offsets && (size_t)a.m <= MEAN_LIMIT * (size_t)a.n_experts))) return SK_NONE;
        const bool two = rows > 16;
        // the formats with the long strips: the one-tile shapes only (see launch_skinny)
        if (Skinny<F>::ONE_TILE && variant != 0 && variant != 200) return SK_NONE;
        if (a.sums && variant != 0 && variant != 200) return SK_NONE;  // the dump exists for the default shapes
        switch (variant) {
        case 0: {
            if (!a.offsets) {
                // one matrix, up to 16 token rows: enough row groups by themselves (a vocabulary projection), or k
                // split over work groups (the workspace has room for the sums)
                if (two) {
                    // 17..32 token rows: only where the tile kernel's 32 x 32 tiles leave half the chip idle (fewer
                    // than 8192 weight rows) and k is long enough to split
                    // (and only from 2^25 weights on: 4096 x 4096 at 17 / 32 rows 13.7 / 16.1 us against 12.7 / 12.8)
                    if (a.n >= 8192 || !has_partial || skinny_splits(a.n, a.k) < 2 || (uint64_t)a.n * a.k < (1ull << 25))
                        return SK_NONE;
                    return Skinny<F>::ONE_TILE ? SK_1_4_SPLIT : SK_2_2_SPLIT;
                }
                if ((size_t)((a.n + 127) / 128) >= 2 * (size_t)device_cus()) return SK_1_4;
                return (has_partial && skinny_splits(a.n, a.k) >= 2) ? SK_1_4_SPLIT : SK_NONE;
            }
            const bool many = (size_t)((a.n + 127) / 128) * a.n_experts >= 2 * (size_t)device_cus();
            // two token tiles: only with many row groups and a mean of at most 20 rows per expert
            if (two) {
                // one tile per work group: a group of 17..32 rows takes a second pass over its expert's weights (the
                // launch's second layer of work groups; those of the smaller groups exit at once).  8 experts of
                // 14336 x 4096, 11..23 rows: Q6_K 152 us, Q8_0 155 against 195 / 227 on the tile kernel; a pass costs
                // 117 / 8 us per expert, so up to a mean of 17 rows (two passes for about half the experts).
                if (Skinny<F>::ONE_TILE) {
                    if ((size_t)a.m > 17 * (size_t)a.n_experts) return SK_NONE;
                    if (many) return SK_1_4;
                    // few row groups per expert (one work group per compute unit in the first pass): the second
                    // pass's work groups would double up on some compute units and set the time; with each expert's
                    // k in two halves the launch spreads evenly
                    const bool can_split = has_partial && a.n <= SKINNY_GROUPED_SPLIT_MAX_N && a.k % 1024 == 0 &&
                                           (size_t)((a.n + 127) / 128) * a.n_experts * SKINNY_GROUPED_SPLITS >= device_cus();
                    return can_split ? SK_1_4_SPLIT : SK_1_8;
                }
                // (a mean of up to 20 rows: 8 experts of 14336 x 4096 with 13..28 rows 92-101 us against 105 + 5 on
                // the tile kernel and its token re-layout)
                if ((size_t)a.m > MEAN_LIMIT * (size_t)a.n_experts) return SK_NONE;
                if (many) return SK_2_2;
                // few row groups per expert: each expert's k in two halves, where that gives every compute unit a
                // work group and the workspace has room for the halves' sums
                const bool can_split = has_partial && a.n <= SKINNY_GROUPED_SPLIT_MAX_N && a.k % 1024 == 0 &&
                                       (size_t)((a.n + 127) / 128) * a.n_experts * SKINNY_GROUPED_SPLITS >= device_cus();
                return can_split ? SK_2_2_SPLIT : SK_NONE;
            }
            if (Skinny<F>::ONE_TILE && !many && has_partial && a.n <= SKINNY_GROUPED_SPLIT_MAX_N && a.k % 1024 == 0 &&
                (size_t)((a.n + 127) / 128) * a.n_experts * SKINNY_GROUPED_SPLITS >= device_cus())
                return SK_1_4_SPLIT;
            // (the debug dump: one shape per token-tile count; every shape adds a result's terms in the same order)
            return (many || a.sums) ? SK_1_4 : SK_1_8;
        }
        case 200: return two && !Skinny<F>::ONE_TILE ? SK_2_2 : SK_1_4;
        case 201: return two ? SK_2_8 : SK_1_16;
        case 203: return two ? SK_W4_2_4 : SK_W4_1_8;
        case 204: return two ? SK_2_2 : SK_1_4;
        case 205: return two ? SK_2_4 : SK_1_8;
        default: return SK_NONE;
        }
    }
    return SK_NONE;
}

// <NT, WAVES, TT, PER>; LDS = PER * 8 * TT * 640 + WAVES * NT * 7 KB
template <class F>
static hipError_t launch_skinny(const GemmArgs &a, const TilePlan &p, hipStream_t stream, int shape) {
    if constexpr (Skinny<F>::OK && Skinny<F>::ONE_TILE) {
        // Q6_K, Q8_0: 8 KB of LDS and more per wave; with chunks of two super-blocks of one token tile two work
        // groups still share a compute unit (75 and 78 KB each)
        switch (shape) {
        case SK_1_4:
        case SK_1_8: return a.sums ? launch_skinny_shape<F, 1, 8, 1, 2, true>(a, p, stream) : launch_skinny_shape<F, 1, 8, 1, 2>(a, p, stream);
        case SK_1_4_SPLIT:
            return a.sums ? launch_skinny_shape<F, 1, 8, 1, 2, true>(a, p, stream, true) : launch_skinny_shape<F, 1, 8, 1, 2>(a, p, stream, true);
        default: break;
        }
    } else if constexpr (Skinny<F>::OK) {
        switch (shape) {
        case SK_1_4: return a.sums ? launch_skinny_shape<F, 1, 8, 1, 4, true>(a, p, stream) : launch_skinny_shape<F, 1, 8, 1, 4>(a, p, stream);
        case SK_2_2: return a.sums ? launch_skinny_shape<F, 1, 8, 2, 2, true>(a, p, stream) : launch_skinny_shape<F, 1, 8, 2, 2>(a, p, stream);
        case SK_1_4_SPLIT:
            return a.sums ? launch_skinny_shape<F, 1, 8, 1, 4, true>(a, p, stream, true) : launch_skinny_shape<F, 1, 8, 1, 4>(a, p, stream, true);
        case SK_2_2_SPLIT:
            return a.sums ? launch_skinny_shape<F, 1, 8, 2, 2, true>(a, p, stream, true) : launch_skinny_shape<F, 1, 8, 2, 2>(a, p, stream, true);
        case SK_1_8: return launch_skinny_shape<F, 1, 8, 1, 8>(a, p, stream);
        case SK_1_16: return launch_skinny_shape<F, 1, 8, 1, 16>(a, p, stream);
        case SK_2_8: return launch_skinny_shape<F, 1, 8, 2, 8>(a, p, stream);
        case SK_2_4: return launch_skinny_shape<F, 1, 8, 2, 4>(a, p, stream);
        case SK_W4_1_8: return launch_skinny_shape<F, 1, 4, 1, 8>(a, p, stream);
        case SK_W4_2_4: return launch_skinny_shape<F, 1, 4, 2, 4>(a, p, stream);
        default: break;
        }
    }
    return hipErrorNotSupported;
}

}  // namespace oxq
