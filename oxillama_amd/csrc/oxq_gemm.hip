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

size_t gemm_workspace_bytes(uint32_t m, uint32_t k) {
    const size_t mpad = ((size_t)m + 127) / 128 * 128, nsb = k / 32;
    return nsb * mpad * (32 + 4 + 2);
}

// One thread per (token, activation block): payload copy, P = da * sum(q), da.
__global__ __launch_bounds__(256) void gemm_prep_acts(const uint8_t *__restrict__ A, uint8_t *__restrict__ q8t,
                                                     float *__restrict__ P, uint16_t *__restrict__ da16, uint32_t m,
                                                     uint32_t mpad, uint32_t nsb) {
    const uint32_t idx = blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= mpad * nsb) return;
    const uint32_t j = idx / mpad, t = idx % mpad;
    u32x4 q0 = {0, 0, 0, 0}, q1 = {0, 0, 0, 0};
    uint32_t dbits = 0;
    if (t < m) {
        const uint8_t *blk = A + ((size_t)t * nsb + j) * Q8_BLOCK_BYTES;
        dbits = ld2(blk);
        q0 = ld16(blk + 2);
        q1 = ld16(blk + 18);
    }
    int s = 0;
    for (int i = 0; i < 4; i++) {
        s = sdot4(q0[i], 0x01010101u, s);
        s = sdot4(q1[i], 0x01010101u, s);
    }
    u32x4 *dst = reinterpret_cast<u32x4 *>(q8t + ((size_t)j * mpad + t) * 32);
    dst[0] = q0;
    dst[1] = q1;
    P[(size_t)j * mpad + t] = h2f(dbits) * (float)s;
    da16[(size_t)j * mpad + t] = (uint16_t)dbits;
}

// Per-lane decode of the scale/min pair of sub-block s of one Q4_K header (decode_scales_mins,
// reference/q4_k.rs:27-49).  hd = the 16 header bytes: d | dmin<<16, scales[0..4], [4..8], [8..12].
__device__ __forceinline__ void q4k_scale_min(const u32x4 hd, uint32_t s, uint32_t &sc, uint32_t &mn) {
    const uint32_t sh = 8 * (s & 3);
    if (s < 4) {
        sc = (hd[1] >> sh) & 63;
        mn = (hd[2] >> sh) & 63;
    } else {
        sc = ((hd[3] >> sh) & 15) | (((hd[1] >> (sh + 6)) & 3) << 4);
        mn = ((hd[3] >> (sh + 4)) & 15) | (((hd[2] >> (sh + 6)) & 3) << 4);
    }
}

// Work group = 4 waves as 2 (tokens) x 2 (weight rows); each wave owns MT x NT MFMA tiles of
// 32 x 32: a (64*MT)-token x (64*NT)-row tile per work group.  Lane l: c = l % 32 is the
// token (A operand) / weight row (B operand) / output column it feeds, h = l / 32 the
// 16-byte half of the 32-byte block.  C layout of the 32x32 MFMAs: register v of lane l
// holds row 8*(v/4) + 4*h + v%4 (token), column c (weight row).
//
// Everything lives in the 256 architectural VGPRs (two waves per SIMD), so MFMA results
// are read by the VALU without accumulator-register copies.  Per super-block the work
// group decodes its rows' 8 scale/min pairs once into LDS as ready-made fp32 factors
// (dsc, -12582912*dsc, -dmin*mn); the f16 token scales of the whole k sit in LDS for the
// life of the work group and enter the accumulate fma as f16 operands.  The min term
// is folded into the same accumulators by one fp32 MFMA per tile and pair of sub-blocks.
// Work groups are numbered so that the token tiles of one set of weight rows run on the
// same XCD at the same time (ids are dealt round-robin to the 8 XCDs), which turns their
// weight reads into L2 hits.
template <int MT, int NT, bool DUMP>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2, 2))) void gemm_q4k_q8_kernel(const uint8_t *__restrict__ W,
                                                            const uint8_t *__restrict__ q8t,
                                                            const float *__restrict__ P,
                                                            const uint16_t *__restrict__ da16,
                                                            float *__restrict__ out, int32_t *__restrict__ sums,
                                                            uint32_t m, uint32_t mpad, uint32_t n, uint32_t k,
                                                            int accumulate, uint32_t m_tiles, uint32_t n_tiles) {
    constexpr int WG_TOK = 64 * MT, WG_ROWS = 64 * NT, MTILES = 2 * MT;
    extern __shared__ uint16_t lds_da[];           // [nsb][MTILES][2 halves][16] f16 token scales
    __shared__ float lds_sc[2][8][3][WG_ROWS];     // [buffer][sub-block][dsc, -MAGIC*dsc, -dmin*mn][row]
    const uint32_t nsb = k / 32, nblk = k / 256, ngrp = nblk * 4;
    const uint32_t tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const uint32_t c = lane & 31, h = lane >> 5;
    const uint32_t wm = wave & 1, wn = wave >> 1;

    const uint32_t xcd = blockIdx.x & 7, loc = blockIdx.x >> 3;
    const uint32_t n_tile = (loc / m_tiles) * 8 + xcd, m_tile = loc % m_tiles;
    if (n_tile >= n_tiles) return;  // whole work group
    const uint32_t m_wg = m_tile * WG_TOK, n_wg = n_tile * WG_ROWS;
    const uint32_t m_wave = m_wg + wm * (32 * MT), n_wave = n_wg + wn * (32 * NT);

    // Token scales of this work group's tokens, permuted so that the 16 values a lane needs
    // for one MFMA tile are 32 contiguous bytes.
    for (uint32_t idx = tid; idx < nsb * WG_TOK; idx += 256) {
        const uint32_t j = idx / WG_TOK, tl = idx % WG_TOK;
        const uint32_t mt = tl >> 5, r = tl & 31;  // r = 8a + 4hh + b
        const uint32_t a = r >> 3, hh = (r >> 2) & 1, b = r & 3;
        lds_da[((j * MTILES + mt) * 2 + hh) * 16 + a * 4 + b] = da16[(size_t)j * mpad + m_wg + tl];
    }

    // Scale decode: thread -> rows (tid % 64) + 64*r, sub-blocks 2*wave and 2*wave + 1.
    const uint8_t *hrow[NT];
    for (int r = 0; r < NT; r++)
        hrow[r] = W + (size_t)min(n_wg + lane + 64 * r, n - 1) * nblk * 144;
    uint32_t hrow_off[NT];
    for (int r = 0; r < NT; r++)
        hrow_off[r] = (min(n_wg + lane + 64 * r, n - 1) - min(n_wg, n - 1)) * (nblk * 144);
    auto decode = [&](const u32x4 (&hd)[NT], uint32_t buf) {
        for (int r = 0; r < NT; r++) {
            const float d = h2f(hd[r][0] & 0xFFFF), dmin = h2f(hd[r][0] >> 16);
#pragma unroll
            for (int e = 0; e < 2; e++) {
                const uint32_t s = 2 * wave + e;
                uint32_t sc, mn;
                q4k_scale_min(hd[r], s, sc, mn);
                const float dsc = d * (float)sc;                       // reference/q4_k.rs:280, exact
                lds_sc[buf][s][0][lane + 64 * r] = dsc;
                lds_sc[buf][s][1][lane + 64 * r] = -(MAGIC_F * dsc);   // exact
                lds_sc[buf][s][2][lane + 64 * r] = -(dmin * (float)mn);  // reference/q4_k.rs:281, exact
            }
        }
    };
    {
        u32x4 hd[NT];
        for (int r = 0; r < NT; r++) hd[r] = ld16(hrow[r]);
        decode(hd, 0);
    }

    v16f acc[MT][NT];
    v16i magic;
    for (int i = 0; i < 16; i++) magic[i] = (int)MAGIC_BITS;
    for (int a = 0; a < MT; a++)
        for (int b = 0; b < NT; b++)
            for (int i = 0; i < 16; i++) acc[a][b][i] = 0.0f;

    // rows past n are clamped for loads and masked at the store
    uint32_t nrow[NT];
    for (int nt = 0; nt < NT; nt++) nrow[nt] = n_wave + nt * 32 + c;
    // Operands come through buffer loads: a wave-uniform descriptor, a fixed 32-bit
    // per-lane offset and a scalar offset that advances with k, so the loop spends no
    // vector instructions on addressing.
    const uint32_t row_bytes = nblk * 144;
    const uint32_t n_base = min(n_wg, n - 1);
    const size_t w_left = (size_t)(n - n_base) * row_bytes;
    const __amdgpu_buffer_rsrc_t rs_w = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<uint8_t *>(W + (size_t)n_base * row_bytes), 0, (int)min(w_left, (size_t)0x7FFFFFFF), BUFFER_FLAGS);
    const __amdgpu_buffer_rsrc_t rs_a =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<uint8_t *>(q8t), 0, (int)(nsb * mpad * 32), BUFFER_FLAGS);
    const __amdgpu_buffer_rsrc_t rs_p =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<float *>(P), 0, (int)(nsb * mpad * 4), BUFFER_FLAGS);
    uint32_t wq_off[NT];  // the lane's 16-byte half of the nibble bytes of group 0 of its row
    for (int nt = 0; nt < NT; nt++) wq_off[nt] = (min(nrow[nt], n - 1) - n_base) * row_bytes + 16 + 16 * h;
    uint32_t aq_off[MT], pq_off[MT];
    for (int mt = 0; mt < MT; mt++) {
        const uint32_t tok = m_wave + mt * 32 + c;  // always < mpad
        aq_off[mt] = tok * 32 + 16 * h;             // the lane's 16 bytes of its token's activation block
        pq_off[mt] = (h * mpad + tok) * 4;          // P of sub-block h of the pair
    }

    struct Ops {
        u32x4 qs[NT];      // 16 nibble bytes per weight row: low nibbles -> sub-block 2g, high -> 2g+1
        u32x4 a[2][MT];    // [sub-block of the pair][token tile] 16 activation bytes
        float pv[MT];      // P of sub-block 2g + h
    };
    // group index G = 4*blk + g; groups past the end re-read the last one (result unused)
    auto fetch = [&](Ops &o, uint32_t G) {
        G = min(G, ngrp - 1);
        const uint32_t w_so = (G >> 2) * 144 + 32 * (G & 3);
        for (int nt = 0; nt < NT; nt++) o.qs[nt] = __builtin_amdgcn_raw_buffer_load_b128(rs_w, wq_off[nt], w_so, 0);
        for (int e = 0; e < 2; e++)
            for (int mt = 0; mt < MT; mt++)
                o.a[e][mt] = __builtin_amdgcn_raw_buffer_load_b128(rs_a, aq_off[mt], (2 * G + e) * mpad * 32, 0);
        for (int mt = 0; mt < MT; mt++)
            o.pv[mt] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(rs_p, pq_off[mt], 2 * G * mpad * 4, 0));
    };

    // One pair of sub-blocks (2g, 2g+1): 2*MT*NT int8 MFMA tiles, each followed by its 32
    // VALU operations; the MFMA of tile t+2 is issued before the VALU work of tile t+1 so
    // that the matrix core runs ahead of the VALU.
    auto compute = [&](const Ops &o, uint32_t blk, uint32_t g, uint32_t buf) {
        constexpr int T = 2 * MT * NT;
        v4i bop[2][NT];
        for (int nt = 0; nt < NT; nt++)
            for (int i = 0; i < 4; i++) {
                bop[0][nt][i] = (int)(o.qs[nt][i] & 0x0F0F0F0Fu);
                bop[1][nt][i] = (int)((o.qs[nt][i] >> 4) & 0x0F0F0F0Fu);
            }
        const uint32_t lrow = wn * (32 * NT) + c;
        auto mfma_tile = [&](int t) {
            const int e = t / (MT * NT), mt = (t / NT) % MT, nt = t % NT;
            v4i aop;
            for (int i = 0; i < 4; i++) aop[i] = (int)o.a[e][mt][i];
            return __builtin_amdgcn_mfma_i32_32x32x32_i8(aop, bop[e][nt], magic, 0, 0, 0);
        };
        v16i dq[2];
        dq[0] = mfma_tile(0);
        if (T > 1) dq[1] = mfma_tile(1);
#pragma unroll
        for (int t = 0; t < T; t++) {
            const int e = t / (MT * NT), mt = (t / NT) % MT, nt = t % NT;
            const uint32_t s = 2 * g + e, j = blk * 8 + s;
            const float dsc = lds_sc[buf][s][0][lrow + nt * 32];
            const float nc2 = lds_sc[buf][s][1][lrow + nt * 32];
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
                    if (row < m && nrow[nt] < n)
                        sums[((size_t)row * n + nrow[nt]) * nsb + j] = (int)(dbits - MAGIC_BITS);
                }
            }
            if (t + 2 < T) dq[t & 1] = mfma_tile(t + 2);
            if (e == 1) {
                // min term of sub-blocks 2g (lanes h = 0) and 2g+1 (lanes h = 1):
                // acc[token][row] += P[token][s] * (-dmin*mn)[row][s], contracted over the pair
                const float qv = lds_sc[buf][2 * g + h][2][lrow + nt * 32];
                acc[mt][nt] = __builtin_amdgcn_mfma_f32_32x32x2f32(o.pv[mt], qv, acc[mt][nt], 0, 0, 0);
            }
        }
    };

    Ops ops0, ops1;
    fetch(ops0, 0);
    __syncthreads();

    for (uint32_t blk = 0; blk < nblk; blk++) {
        const uint32_t buf = blk & 1;
        const uint32_t nxt = min(blk + 1, nblk - 1);  // last trip: harmless re-read
        u32x4 hd[NT];
        for (int r = 0; r < NT; r++) hd[r] = __builtin_amdgcn_raw_buffer_load_b128(rs_w, hrow_off[r], nxt * 144, 0);
        fetch(ops1, blk * 4 + 1);
        compute(ops0, blk, 0, buf);
        fetch(ops0, blk * 4 + 2);
        compute(ops1, blk, 1, buf);
        fetch(ops1, blk * 4 + 3);
        compute(ops0, blk, 2, buf);
        fetch(ops0, blk * 4 + 4);
        compute(ops1, blk, 3, buf);
        decode(hd, buf ^ 1);
        __syncthreads();
    }

    for (int mt = 0; mt < MT; mt++)
        for (int nt = 0; nt < NT; nt++) {
            if (nrow[nt] >= n) continue;
#pragma unroll
            for (int i = 0; i < 16; i++) {
                const uint32_t row = m_wave + mt * 32 + 8 * (i >> 2) + 4 * h + (i & 3);
                if (row < m) {
                    float *o = out + (size_t)row * n + nrow[nt];
                    *o = accumulate ? *o + acc[mt][nt][i] : acc[mt][nt][i];
                }
            }
        }
}

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

template <int MT, int NT>
static hipError_t launch_tile_variant(const GemmArgs &a, const uint8_t *q8t, const float *P, const uint16_t *da16,
                                      uint32_t mpad, hipStream_t stream) {
    const uint32_t m_tiles = mpad / (64 * MT), n_tiles = (a.n + 64 * NT - 1) / (64 * NT);
    const dim3 grid(8 * ((n_tiles + 7) / 8) * m_tiles);
    const size_t lds = (size_t)(a.k / 32) * (64 * MT) * 2;
    hipError_t e = hipSuccess;
    if (lds > 32 * 1024) {  // beyond the default dynamic LDS limit: opt in (up to the 160 KB of a CU)
        e = a.sums ? hipFuncSetAttribute(reinterpret_cast<const void *>(&gemm_q4k_q8_kernel<MT, NT, true>),
                                         hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds)
                   : hipFuncSetAttribute(reinterpret_cast<const void *>(&gemm_q4k_q8_kernel<MT, NT, false>),
                                         hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (e != hipSuccess) return e;
    }
    if (a.sums)
        hipLaunchKernelGGL((gemm_q4k_q8_kernel<MT, NT, true>), grid, dim3(256), lds, stream, a.W, q8t, P, da16, a.out,
                           a.sums, a.m, mpad, a.n, a.k, a.accumulate, m_tiles, n_tiles);
    else
        hipLaunchKernelGGL((gemm_q4k_q8_kernel<MT, NT, false>), grid, dim3(256), lds, stream, a.W, q8t, P, da16, a.out,
                           a.sums, a.m, mpad, a.n, a.k, a.accumulate, m_tiles, n_tiles);
    return hipGetLastError();
}

static hipError_t launch_tiles(const GemmArgs &a, const uint8_t *q8t, const float *P, const uint16_t *da16,
                               uint32_t mpad, hipStream_t stream) {
    switch (g_gemm_variant) {
    case 1: return launch_tile_variant<2, 1>(a, q8t, P, da16, mpad, stream);
    case 2: return launch_tile_variant<1, 2>(a, q8t, P, da16, mpad, stream);
    case 3: return launch_tile_variant<2, 2>(a, q8t, P, da16, mpad, stream);
    case 4: return launch_tile_variant<1, 1>(a, q8t, P, da16, mpad, stream);
    default: return launch_tile_variant<2, 2>(a, q8t, P, da16, mpad, stream);
    }
}

bool gemm_uses_tiles(uint32_t type, uint32_t m, uint32_t k) {
    // LDS holds the f16 token scales of up to 128 tokens for the whole k (k/32 * 256 bytes)
    // beside 24 KB of decoded weight scales; up to k = 8192 two work groups share a CU
    return type == OXQ_TYPE_Q4_K && m >= 8 && (size_t)(k / 32) * 256 <= 128 * 1024;
}

hipError_t launch_gemm_q8(uint32_t type, const GemmArgs &a, hipStream_t stream) {
    if (!gemm_uses_tiles(type, a.m, a.k) || a.workspace == nullptr) return gemm_by_rows(type, a, stream);
    const uint32_t mpad = (a.m + 127) / 128 * 128, nsb = a.k / 32;
    uint8_t *q8t = a.workspace;
    float *P = reinterpret_cast<float *>(q8t + (size_t)nsb * mpad * 32);
    uint16_t *da16 = reinterpret_cast<uint16_t *>(q8t + (size_t)nsb * mpad * 36);
    hipLaunchKernelGGL(gemm_prep_acts, dim3((mpad * nsb + 255) / 256), dim3(256), 0, stream, a.A, q8t, P, da16, a.m,
                       mpad, nsb);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return e;
    return launch_tiles(a, q8t, P, da16, mpad, stream);
}

}  // namespace oxq
