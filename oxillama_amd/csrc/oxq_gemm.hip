// Batched (prefill) form of the fused matvec on gfx950:
//   out[m x n] (+)= A_q8[m rows of Q8_0 blocks] x W[n x k]^T
// i.e. m fused matvecs over the same weight blocks (the reference's gemm is exactly
// that loop, crates/oxillama-quant/src/reference/q4_k.rs:186-201, with
// matvec_q8_fused's arithmetic, :218-333).
//
// Q4_K runs on the int8 matrix cores.  One v_mfma_i32_32x32x32_i8 contracts one
// 32-weight sub-block of 32 weight rows against the matching Q8_0 block of 32
// tokens, so every int32 result is exactly one "group sum" I[m][n][s] of the
// matvec.  The fp32 value is then
//   y[m][n] = sum_s da[m][s] * (d_n*sc_ns) * I  -  sum_s (da[m][s]*S[m][s]) * (dmin_n*mn_ns)
// (S = sum of the block's int8 activations).
//  * first sum: the MFMA adds into the constant 0x4B400000 (= 12582912.0f), so the
//    int32 result read as a float is 12582912 + I exactly; one fma with the per-lane
//    constants dsc and -12582912*dsc (exact: dsc has <= 17 significant bits) gives
//    fl(dsc * I) -- the rounding of the reference's `da * dot as f32` -- without an
//    int->float conversion, and a second fma with the token's f16 scale accumulates.
//    Two VALU operations per (token, weight row, sub-block): that, not the matrix
//    core, bounds this kernel.
//  * second sum: a rank-(k/32) fp32 product, added into the same accumulators with
//    v_mfma_f32_32x32x2_f32 on P[m][s] = da*S and -dmin*mn while the VALU works on
//    other tiles.
// A small preparation kernel lays the activations out once per call: int8 payload
// tiled [k/32][m][32] (so every MFMA operand load is one aligned, contiguous KB),
// P as fp32 [k/32][m], da as f16 [k/32][m].
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
// A 256-weight super-block is walked as 4 groups of 2 sub-blocks; for group g lane (c, h)
// loads the 16 bytes at QS_OFF + 32*g + 16*h of its row's block.

// Q4_K (reference/q4_k.rs:27-102): those 16 bytes carry weights 16h..16h+15 of sub-block 2g
// in the low nibbles and of sub-block 2g+1 in the high nibbles.
struct TileQ4K {
    static constexpr uint32_t TYPE = OXQ_TYPE_Q4_K, BLOCK_BYTES = 144, QS_OFF = 16;
    static constexpr bool HAS_MIN = true;
    static constexpr int ACT_PERM = 0;  // activation bytes stay in column order
    // hd = the 16 header bytes: d | dmin<<16, scales[0..4], [4..8], [8..12] (decode_scales_mins, :27-49)
    static __device__ __forceinline__ void scales(const u32x4 hd, uint32_t s, float &dsc, float &qneg) {
        const uint32_t sh = 8 * (s & 3);
        uint32_t sc, mn;
        if (s < 4) {
            sc = (hd[1] >> sh) & 63;
            mn = (hd[2] >> sh) & 63;
        } else {
            sc = ((hd[3] >> sh) & 15) | (((hd[1] >> (sh + 6)) & 3) << 4);
            mn = ((hd[3] >> (sh + 4)) & 15) | (((hd[2] >> (sh + 6)) & 3) << 4);
        }
        dsc = h2f(hd[0] & 0xFFFF) * (float)sc;       // reference/q4_k.rs:280, exact
        qneg = -(h2f(hd[0] >> 16) * (float)mn);      // reference/q4_k.rs:281, exact
    }
    static __device__ __forceinline__ void operands(const u32x4 qs, v4i (&bop)[2]) {
        for (int i = 0; i < 4; i++) {
            bop[0][i] = (int)(qs[i] & 0x0F0F0F0Fu);
            bop[1][i] = (int)((qs[i] >> 4) & 0x0F0F0F0Fu);
        }
    }
};

// IQ4_XS (reference/iq4_xs.rs:47-97): the 16 bytes are the whole sub-block 2g+h, byte j =
// codebook indices of weights 2j (low nibble) and 2j+1 (high).  The two halves of the wave
// trade 8 bytes (v_permlane32_swap) so that lane (c, h) ends up with bytes 8h..8h+7 of
// sub-block 2g and of sub-block 2g+1; the table lookup then yields weights
// 16h + {0,2,4,6, 1,3,5,7, 8,10,12,14, 9,11,13,15}, and the activation bytes are stored in
// that same order by the preparation kernel (ACT_PERM).
struct TileIQ4XS {
    static constexpr uint32_t TYPE = OXQ_TYPE_IQ4_XS, BLOCK_BYTES = 136, QS_OFF = 8;
    static constexpr bool HAS_MIN = false;
    static constexpr int ACT_PERM = 1;
    // hd = the first 16 bytes: d | scales_h<<16, scales_l, (qs...) (unpack_sub_scale, :47-53)
    static __device__ __forceinline__ void scales(const u32x4 hd, uint32_t s, float &dsc, float &qneg) {
        const uint32_t ls = ((hd[1] >> (4 * s)) & 15) | ((((hd[0] >> 16) >> (2 * s)) & 3) << 4);
        dsc = h2f(hd[0] & 0xFFFF) * (float)((int)ls - 32);  // reference/iq4_xs.rs:81, exact
        qneg = 0.0f;
    }
    static __device__ __forceinline__ void operands(const u32x4 qs, v4i (&bop)[2]) {
        const auto s02 = __builtin_amdgcn_permlane32_swap(qs[0], qs[2], false, false);
        const auto s13 = __builtin_amdgcn_permlane32_swap(qs[1], qs[3], false, false);
        const uint32_t x[2][2] = {{s02[0], s13[0]}, {s02[1], s13[1]}};
        for (int e = 0; e < 2; e++)
            for (int i = 0; i < 2; i++) {
                bop[e][2 * i] = (int)FmtIQ4XS::lut4(x[e][i] & 0x0F0F0F0Fu);
                bop[e][2 * i + 1] = (int)FmtIQ4XS::lut4((x[e][i] >> 4) & 0x0F0F0F0Fu);
            }
    }
};

// One thread per (token, activation block): payload copy (optionally permuted inside each
// 16-byte half to the order the weight lookup produces), P = da * sum(q), da.
template <int PERM>
__global__ __launch_bounds__(256) void gemm_prep_acts(const uint8_t *__restrict__ A, uint8_t *__restrict__ q8t,
                                                     float *__restrict__ P, uint16_t *__restrict__ da16, uint32_t m,
                                                     uint32_t mpad, uint32_t nsb) {
    const uint32_t idx = blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= mpad * nsb) return;
    const uint32_t j = idx / mpad, t = idx % mpad;
    u32x4 q[2] = {{0, 0, 0, 0}, {0, 0, 0, 0}};
    uint32_t dbits = 0;
    if (t < m) {
        const uint8_t *blk = A + ((size_t)t * nsb + j) * Q8_BLOCK_BYTES;
        dbits = ld2(blk);
        q[0] = ld16(blk + 2);
        q[1] = ld16(blk + 18);
    }
    int s = 0;
    for (int i = 0; i < 4; i++) {
        s = sdot4(q[0][i], 0x01010101u, s);
        s = sdot4(q[1][i], 0x01010101u, s);
    }
    if (PERM) {
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
    da16[(size_t)j * mpad + t] = (uint16_t)dbits;
}

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
template <class F, int MT, int NT, int WM, int DIST, bool DUMP>
__device__ __forceinline__ void gemm_tile_body(
    const uint8_t *__restrict__ W, const uint8_t *__restrict__ q8t, const float *__restrict__ P,
    const uint16_t *__restrict__ da16, float *__restrict__ out, int32_t *__restrict__ sums, uint32_t m, uint32_t mpad,
    uint32_t n, uint32_t k, int accumulate, uint32_t m_tiles, uint32_t n_tiles, const int32_t *__restrict__ offsets,
    size_t w_stride) {
    constexpr int WN = 4 / WM;
    constexpr int WG_TOK = 32 * MT * WM, WG_ROWS = 32 * NT * WN, MTILES = MT * WM;
    constexpr int NP = F::HAS_MIN ? 3 : 2;
    constexpr int W_ROWS = 32 * NT;                  // weight rows of one wave
    constexpr int LPR = 64 / W_ROWS, SPL = 8 / LPR;  // scale decode: lanes per row, sub-blocks per lane
    static_assert(NT <= 2 && (DIST == 1 || DIST == 2 || DIST == 4), "tile configuration");
    extern __shared__ uint16_t lds_da[];            // [nsb][MTILES][2 halves][16] f16 token scales
    __shared__ float lds_sc[4][8][NP][W_ROWS];      // [wave][sub-block][dsc, -MAGIC*dsc, -dmin*mn][row of the wave]
    const uint32_t nsb = k / 32, nblk = k / 256, ngrp = nblk * 4;
    const uint32_t tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const uint32_t c = lane & 31, h = lane >> 5;
    const uint32_t wm = wave % WM, wn = wave / WM;

    const uint32_t xcd = blockIdx.x & 7, loc = blockIdx.x >> 3;
    const uint32_t n_tile = (loc / m_tiles) * 8 + xcd, m_tile = loc % m_tiles;
    uint32_t row0 = 0, row_end = m;
    if (offsets) {
        row0 = (uint32_t)offsets[blockIdx.y];
        row_end = (uint32_t)offsets[blockIdx.y + 1];
        W += (size_t)blockIdx.y * w_stride;
    }
    if (n_tile >= n_tiles || row0 + m_tile * WG_TOK >= row_end) return;  // whole work group
    const uint32_t m_wg = row0 + m_tile * WG_TOK, n_wg = n_tile * WG_ROWS;
    const uint32_t m_wave = m_wg + wm * (32 * MT), n_wave = n_wg + wn * (32 * NT);

    // Token scales of this work group's tokens, permuted so that the 16 values a lane needs
    // for one MFMA tile are 32 contiguous bytes.
    for (uint32_t idx = tid; idx < nsb * WG_TOK; idx += 256) {
        const uint32_t j = idx / WG_TOK, tl = idx % WG_TOK;
        const uint32_t mt = tl >> 5, r = tl & 31;  // r = 8a + 4hh + b
        const uint32_t a = r >> 3, hh = (r >> 2) & 1, b = r & 3;
        lds_da[((j * MTILES + mt) * 2 + hh) * 16 + a * 4 + b] = da16[(size_t)j * mpad + m_wg + tl];
    }

    // Operands come through buffer loads: a wave-uniform descriptor, a fixed 32-bit
    // per-lane offset and a scalar offset that advances with k, so the loop spends no
    // vector instructions on addressing.  Rows past n are clamped for loads and masked
    // at the store.
    const uint32_t row_bytes = nblk * F::BLOCK_BYTES;
    const uint32_t n_base = min(n_wg, n - 1);
    const size_t w_left = (size_t)(n - n_base) * row_bytes;
    const __amdgpu_buffer_rsrc_t rs_w = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<uint8_t *>(W + (size_t)n_base * row_bytes), 0, (int)min(w_left, (size_t)0x7FFFFFFF), BUFFER_FLAGS);
    const __amdgpu_buffer_rsrc_t rs_a =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<uint8_t *>(q8t), 0, (int)(nsb * mpad * 32), BUFFER_FLAGS);
    const __amdgpu_buffer_rsrc_t rs_p =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<float *>(P), 0, (int)(nsb * mpad * 4), BUFFER_FLAGS);

    // Scale decode, per wave for its own rows (no work-group barrier in the k loop): lane ->
    // row lane % W_ROWS, sub-blocks SPL * (lane / W_ROWS) + 0..SPL-1.  The wave writes the
    // factors of the next super-block after its last read of the current ones.
    const uint32_t drow = lane % W_ROWS, ds0 = SPL * (lane / W_ROWS);
    const uint32_t hrow_off = (min(n_wave + drow, n - 1) - n_base) * row_bytes;
    auto decode = [&](const u32x4 hd) {
#pragma unroll
        for (int e = 0; e < SPL; e++) {
            const uint32_t s = ds0 + e;
            float dsc, qneg;
            F::scales(hd, s, dsc, qneg);
            lds_sc[wave][s][0][drow] = dsc;
            lds_sc[wave][s][1][drow] = -(MAGIC_F * dsc);  // exact
            if (F::HAS_MIN) lds_sc[wave][s][NP - 1][drow] = qneg;
        }
    };
    decode(__builtin_amdgcn_raw_buffer_load_b128(rs_w, hrow_off, 0, 0));

    v16f acc[MT][NT];
    v16i magic;
    for (int i = 0; i < 16; i++) magic[i] = (int)MAGIC_BITS;
    for (int a = 0; a < MT; a++)
        for (int b = 0; b < NT; b++)
            for (int i = 0; i < 16; i++) acc[a][b][i] = 0.0f;

    uint32_t nrow[NT], wq_off[NT];  // wq_off: the lane's 16 bytes of group 0 of its row
    for (int nt = 0; nt < NT; nt++) {
        nrow[nt] = n_wave + nt * 32 + c;
        wq_off[nt] = (min(nrow[nt], n - 1) - n_base) * row_bytes + F::QS_OFF + 16 * h;
    }
    uint32_t aq_off[MT], pq_off[MT];
    for (int mt = 0; mt < MT; mt++) {
        const uint32_t tok = m_wave + mt * 32 + c;  // always < mpad
        aq_off[mt] = tok * 32 + 16 * h;             // the lane's 16 bytes of its token's activation block
        pq_off[mt] = (h * mpad + tok) * 4;          // P of sub-block h of the pair
    }

    struct Ops {
        u32x4 a[2][MT];  // [sub-block of the pair][token tile] 16 activation bytes
        float pv[MT];    // P of sub-block 2g + h
    };
    // group index G = 4*blk + g; groups past the end re-read the last one (result unused)
    auto fetch_w = [&](u32x4 (&qs)[NT], uint32_t G) {
        G = min(G, ngrp - 1);
        const uint32_t w_so = (G >> 2) * F::BLOCK_BYTES + 32 * (G & 3);
        for (int nt = 0; nt < NT; nt++) qs[nt] = __builtin_amdgcn_raw_buffer_load_b128(rs_w, wq_off[nt], w_so, 0);
    };
    auto fetch_a = [&](Ops &o, uint32_t G) {
        G = min(G, ngrp - 1);
        for (int e = 0; e < 2; e++)
            for (int mt = 0; mt < MT; mt++)
                o.a[e][mt] = __builtin_amdgcn_raw_buffer_load_b128(rs_a, aq_off[mt], (2 * G + e) * mpad * 32, 0);
        if (F::HAS_MIN)
            for (int mt = 0; mt < MT; mt++)
                o.pv[mt] = __builtin_bit_cast(
                    float, __builtin_amdgcn_raw_buffer_load_b32(rs_p, pq_off[mt], 2 * G * mpad * 4, 0));
    };

    // One pair of sub-blocks (2g, 2g+1): 2*MT*NT int8 MFMA tiles, each followed by its 32
    // VALU operations; the MFMA of tile t+2 is issued before the VALU work of tile t+1 so
    // that the matrix core runs ahead of the VALU.
    auto compute = [&](const u32x4 (&qs)[NT], const Ops &o, uint32_t blk, uint32_t g) {
        constexpr int T = 2 * MT * NT;
        v4i bop[NT][2];
        for (int nt = 0; nt < NT; nt++) F::operands(qs[nt], bop[nt]);
        auto mfma_tile = [&](int t) {
            const int e = t / (MT * NT), mt = (t / NT) % MT, nt = t % NT;
            v4i aop;
            for (int i = 0; i < 4; i++) aop[i] = (int)o.a[e][mt][i];
            return __builtin_amdgcn_mfma_i32_32x32x32_i8(aop, bop[nt][e], magic, 0, 0, 0);
        };
        v16i dq[2];
        dq[0] = mfma_tile(0);
        if (T > 1) dq[1] = mfma_tile(1);
#pragma unroll
        for (int t = 0; t < T; t++) {
            const int e = t / (MT * NT), mt = (t / NT) % MT, nt = t % NT;
            const uint32_t s = 2 * g + e, j = blk * 8 + s;
            const float dsc = lds_sc[wave][s][0][nt * 32 + c];
            const float nc2 = lds_sc[wave][s][1][nt * 32 + c];
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
                    if (row < row_end && nrow[nt] < n)
                        sums[((size_t)row * n + nrow[nt]) * nsb + j] = (int)(dbits - MAGIC_BITS);
                }
            }
            if (t + 2 < T) dq[t & 1] = mfma_tile(t + 2);
            if (F::HAS_MIN && e == 1) {
                // min term of sub-blocks 2g (lanes h = 0) and 2g+1 (lanes h = 1):
                // acc[token][row] += P[token][s] * (-dmin*mn)[row][s], contracted over the pair
                const float qv = lds_sc[wave][2 * g + h][NP - 1][nt * 32 + c];
                acc[mt][nt] = __builtin_amdgcn_mfma_f32_32x32x2f32(o.pv[mt], qv, acc[mt][nt], 0, 0, 0);
            }
        }
    };

    u32x4 wring[DIST][NT];
    Ops ops0, ops1;
#pragma unroll
    for (int d = 0; d < DIST; d++) fetch_w(wring[d], d);
    fetch_a(ops0, 0);
    __syncthreads();

    for (uint32_t blk = 0; blk < nblk; blk++) {
        const uint32_t nxt = min(blk + 1, nblk - 1);  // last trip: harmless re-read
        const u32x4 hd = __builtin_amdgcn_raw_buffer_load_b128(rs_w, hrow_off, nxt * F::BLOCK_BYTES, 0);
#pragma unroll
        for (int g = 0; g < 4; g++) {
            u32x4 qs[NT];
            for (int nt = 0; nt < NT; nt++) qs[nt] = wring[g % DIST][nt];
            fetch_w(wring[g % DIST], blk * 4 + g + DIST);  // slot consumed: refill it DIST groups ahead
            if (g & 1) {
                fetch_a(ops0, blk * 4 + g + 1);
                compute(qs, ops1, blk, g);
            } else {
                fetch_a(ops1, blk * 4 + g + 1);
                compute(qs, ops0, blk, g);
            }
        }
        __builtin_amdgcn_wave_barrier();  // the wave's reads of this super-block's factors come first
        decode(hd);
        __builtin_amdgcn_wave_barrier();
    }

    for (int mt = 0; mt < MT; mt++)
        for (int nt = 0; nt < NT; nt++) {
            if (nrow[nt] >= n) continue;
#pragma unroll
            for (int i = 0; i < 16; i++) {
                const uint32_t row = m_wave + mt * 32 + 8 * (i >> 2) + 4 * h + (i & 3);
                if (row < row_end) {
                    float *o = out + (size_t)row * n + nrow[nt];
                    *o = accumulate ? *o + acc[mt][nt][i] : acc[mt][nt][i];
                }
            }
        }
}

// The kernel proper, compiled for a fixed number of waves per SIMD (OCC = 2: up to 256 VGPRs,
// OCC = 3: up to 168): the register budget decides how far the compiler lets loads and MFMAs
// run ahead of their use.
#define OXQ_TILE_KERNEL(NAME, OCC)                                                                                   \
    template <class F, int MT, int NT, int WM, int DIST, bool DUMP>                                                 \
    __global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(OCC, OCC))) void NAME(                      \
        const uint8_t *__restrict__ W, const uint8_t *__restrict__ q8t, const float *__restrict__ P,                \
        const uint16_t *__restrict__ da16, float *__restrict__ out, int32_t *__restrict__ sums, uint32_t m,         \
        uint32_t mpad, uint32_t n, uint32_t k, int accumulate, uint32_t m_tiles, uint32_t n_tiles,                  \
        const int32_t *__restrict__ offsets, size_t w_stride) {                                                     \
        gemm_tile_body<F, MT, NT, WM, DIST, DUMP>(W, q8t, P, da16, out, sums, m, mpad, n, k, accumulate, m_tiles,   \
                                                  n_tiles, offsets, w_stride);                                      \
    }
OXQ_TILE_KERNEL(gemm_tile_kernel, 2)
OXQ_TILE_KERNEL(gemm_tile_kernel_occ3, 3)
#undef OXQ_TILE_KERNEL

// One fused matvec per activation row: every format other than Q4_K, and Q4_K shapes the
// tile kernel does not take.
static hipError_t gemm_by_rows(uint32_t type, const GemmArgs &a, hipStream_t stream) {
    const size_t act_row_bytes = (size_t)(a.k / 32) * 34;
    for (uint32_t r = 0; r < a.m; r++) {
        GemvArgs g;
        g.W = a.W;
        g.A = a.A + r * act_row_bytes;
        g.out = a.out + (size_t)r * a.n;
        g.sums = nullptr;
        g.n_rows = a.n;
        g.n_cols = a.k;
        g.accumulate = a.accumulate;
        g.waves_per_cu = 8;
        g.rows_per_batch = 0;
        g.waves_per_row = 0;
        hipError_t e = launch_gemv_q8(type, g, stream);
        if (e != hipSuccess) return e;
    }
    return hipSuccess;
}

int g_gemm_variant = 0;  // tuning: 0 = default

struct TilePlan {
    const uint8_t *q8t;
    const float *P;
    const uint16_t *da16;
    uint32_t mpad;
};

template <class F, int MT, int NT, int WM, int DIST, bool DUMP, int OCC = 2>
static hipError_t launch_tile(const GemmArgs &a, const TilePlan &p, hipStream_t stream) {
    constexpr uint32_t WG_TOK = 32 * MT * WM, WG_ROWS = 32 * NT * (4 / WM);
    const uint32_t rows = a.offsets ? a.max_rows : a.m;
    const uint32_t m_tiles = (rows + WG_TOK - 1) / WG_TOK, n_tiles = (a.n + WG_ROWS - 1) / WG_ROWS;
    const dim3 grid(8 * ((n_tiles + 7) / 8) * m_tiles, a.offsets ? a.n_experts : 1);
    const size_t lds = (size_t)(a.k / 32) * WG_TOK * 2;
    auto kern = OCC == 3 ? &gemm_tile_kernel_occ3<F, MT, NT, WM, DIST, DUMP> : &gemm_tile_kernel<F, MT, NT, WM, DIST, DUMP>;
    if (lds > 32 * 1024) {  // beyond the default dynamic LDS limit: opt in (up to the 160 KB of a CU)
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kern),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (e != hipSuccess) return e;
    }
    hipLaunchKernelGGL(kern, grid, dim3(256), lds, stream, a.W, p.q8t, p.P, p.da16, a.out, a.sums, a.m, p.mpad, a.n,
                       a.k, a.accumulate, m_tiles, n_tiles, a.offsets, a.w_stride);
    return hipGetLastError();
}

// Tile shape by use: prefill (many tokens) takes 128 x 128 work-group tiles; few tokens
// (a mixture-of-experts group, a short prompt) take 32 tokens x 256 rows with the weight
// bytes fetched further ahead, because that case is bound by the weight stream from HBM.
template <class F>
static hipError_t launch_tiles(const GemmArgs &a, const TilePlan &p, hipStream_t stream) {
    const uint32_t rows = a.offsets ? a.max_rows : a.m;
    if (a.sums)
        return rows > 32 ? launch_tile<F, 2, 2, 2, 1, true>(a, p, stream) : launch_tile<F, 1, 2, 1, 2, true>(a, p, stream);
    switch (g_gemm_variant) {
    case 1: return launch_tile<F, 2, 1, 2, 1, false>(a, p, stream);
    case 2: return launch_tile<F, 1, 2, 2, 1, false>(a, p, stream);
    case 3: return launch_tile<F, 2, 2, 2, 1, false>(a, p, stream);
    case 4: return launch_tile<F, 2, 2, 2, 2, false>(a, p, stream);
    case 5: return launch_tile<F, 2, 1, 2, 1, false, 3>(a, p, stream);
    case 6: return launch_tile<F, 1, 2, 2, 1, false, 3>(a, p, stream);
    case 7: return launch_tile<F, 1, 1, 2, 1, false, 3>(a, p, stream);
    case 11: return launch_tile<F, 1, 2, 1, 1, false>(a, p, stream);
    case 12: return launch_tile<F, 1, 2, 1, 2, false>(a, p, stream);
    case 13: return launch_tile<F, 1, 2, 1, 4, false>(a, p, stream);
    case 14: return launch_tile<F, 1, 1, 1, 2, false>(a, p, stream);
    case 15: return launch_tile<F, 1, 1, 1, 4, false>(a, p, stream);
    case 16: return launch_tile<F, 2, 1, 1, 2, false>(a, p, stream);
    default:
        if (rows > 32) return launch_tile<F, 2, 2, 2, 1, false>(a, p, stream);
        // few tokens: 256-row tiles unless that leaves compute units without a work group
        if ((size_t)((a.n + 255) / 256) * (a.offsets ? a.n_experts : 1) >= device_cus())
            return launch_tile<F, 1, 2, 1, 2, false>(a, p, stream);
        return launch_tile<F, 1, 1, 1, 2, false>(a, p, stream);
    }
}

size_t gemm_workspace_bytes(uint32_t m, uint32_t k) {
    // token rows are padded so that a 128-token tile starting at any row stays inside
    const size_t mpad = ((size_t)m + 127) / 128 * 128 + 128, nsb = k / 32;
    return nsb * mpad * (32 + 4 + 2);
}

bool gemm_uses_tiles(uint32_t type, uint32_t m, uint32_t k) {
    // LDS holds the f16 token scales of up to 128 tokens for the whole k (k/32 * 256 bytes)
    // beside up to 24 KB of decoded weight scales; up to k = 8192 two work groups share a CU
    return (type == OXQ_TYPE_Q4_K || type == OXQ_TYPE_IQ4_XS) && m >= 8 && (size_t)(k / 32) * 256 <= 128 * 1024 &&
           gemm_workspace_bytes(m, k) < 0x7FFFFFFFull;
}

hipError_t launch_gemm_q8(uint32_t type, const GemmArgs &a, hipStream_t stream) {
    if (!gemm_uses_tiles(type, a.m, a.k) || a.workspace == nullptr) {
        if (a.offsets) return hipErrorInvalidValue;  // grouped form exists for the tile kernel only
        return gemm_by_rows(type, a, stream);
    }
    const uint32_t mpad = (a.m + 127) / 128 * 128 + 128, nsb = a.k / 32;
    uint8_t *q8t = a.workspace;
    float *P = reinterpret_cast<float *>(q8t + (size_t)nsb * mpad * 32);
    uint16_t *da16 = reinterpret_cast<uint16_t *>(q8t + (size_t)nsb * mpad * 36);
    const dim3 pgrid((mpad * nsb + 255) / 256);
    if (type == OXQ_TYPE_IQ4_XS)
        hipLaunchKernelGGL(gemm_prep_acts<1>, pgrid, dim3(256), 0, stream, a.A, q8t, P, da16, a.m, mpad, nsb);
    else
        hipLaunchKernelGGL(gemm_prep_acts<0>, pgrid, dim3(256), 0, stream, a.A, q8t, P, da16, a.m, mpad, nsb);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return e;
    const TilePlan plan = {q8t, P, da16, mpad};
    return type == OXQ_TYPE_IQ4_XS ? launch_tiles<TileIQ4XS>(a, plan, stream) : launch_tiles<TileQ4K>(a, plan, stream);
}

}  // namespace oxq
