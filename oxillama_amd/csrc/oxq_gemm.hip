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
//  * second sum: a rank-(k/32) fp32 product, done with v_mfma_f32_32x32x2_f32 on
//    P[m][s] = da*S and -dmin*mn, in the shadow of the VALU work.
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

// Work group = 4 waves as 2 (tokens) x 2 (weight rows); each wave owns a 64 x (32*NT)
// tile = 2 x NT MFMA tiles of 32 x 32.  Lane l: c = l % 32 is the token (A operand) /
// weight row (B operand) / output column it feeds, h = l / 32 the 16-byte half of
// the 32-byte block.  C layout of the 32x32 MFMAs: register v of lane l holds row
// 8*(v/4) + 4*h + v%4 (token), column c (weight row).
// Operands are fetched DIST 64-column groups ahead into a ring of register slots
// (DIST divides 4, so the slot of a group is fixed at compile time).
template <int NT, int DIST, bool DUMP>
__global__ __launch_bounds__(256) void gemm_q4k_q8_kernel(const uint8_t *__restrict__ W,
                                                         const uint8_t *__restrict__ q8t,
                                                         const float *__restrict__ P,
                                                         const uint16_t *__restrict__ da16,
                                                         float *__restrict__ out, int32_t *__restrict__ sums,
                                                         uint32_t m, uint32_t mpad, uint32_t n, uint32_t k,
                                                         int accumulate) {
    static_assert(DIST == 1 || DIST == 2 || DIST == 4, "prefetch distance in groups");
    extern __shared__ uint16_t lds_da[];  // [nsb][4 m-tiles][2 halves][16] f16 token scales of this work group
    const uint32_t nsb = k / 32, nblk = k / 256, ngrp = nblk * 4;
    const uint32_t tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const uint32_t c = lane & 31, h = lane >> 5;
    const uint32_t wm = wave & 1, wn = wave >> 1;
    const uint32_t m_wg = blockIdx.x * 128, n_wave = blockIdx.y * (64 * NT) + wn * (32 * NT);
    const uint32_t m_wave = m_wg + wm * 64;

    // Token scales of the 128 tokens of this work group, permuted so that the 16 values a
    // lane needs for one MFMA tile are 32 contiguous bytes.
    for (uint32_t idx = tid; idx < nsb * 128; idx += 256) {
        const uint32_t j = idx >> 7, tl = idx & 127;
        const uint32_t mt = tl >> 5, r = tl & 31;  // r = 8a + 4hh + b
        const uint32_t a = r >> 3, hh = (r >> 2) & 1, b = r & 3;
        lds_da[((j * 4 + mt) * 2 + hh) * 16 + a * 4 + b] = da16[(size_t)j * mpad + m_wg + tl];
    }
    __syncthreads();

    v16f acc[2][NT], acc2[2][NT];
    v16i magic;
    for (int i = 0; i < 16; i++) magic[i] = (int)MAGIC_BITS;
    for (int a = 0; a < 2; a++)
        for (int b = 0; b < NT; b++)
            for (int i = 0; i < 16; i++) {
                acc[a][b][i] = 0.0f;
                acc2[a][b][i] = 0.0f;
            }

    // rows past n are clamped for loads and masked at the store
    uint32_t nrow[NT];
    const uint8_t *wrow[NT];
    for (int nt = 0; nt < NT; nt++) {
        nrow[nt] = n_wave + nt * 32 + c;
        wrow[nt] = W + (size_t)min(nrow[nt], n - 1) * nblk * 144;
    }
    const uint32_t mtok[2] = {m_wave + c, m_wave + 32 + c};  // always < mpad

    struct Slot {
        u32x4 qs[NT];     // 16 nibble bytes per weight row: low nibbles -> sub-block 2g, high -> 2g+1
        u32x4 aop[2][2];  // [half][mt] 16 activation bytes
        float pv[2];      // P of sub-block 2g + h
    };
    Slot slot[DIST];
    u32x4 hdr[NT];
    // group index G = 4*blk + g; groups past the end re-read the last one (result unused)
    auto fill = [&](Slot &sl, uint32_t G) {
        G = min(G, ngrp - 1);
        const uint32_t blk = G >> 2, g = G & 3;
        for (int nt = 0; nt < NT; nt++) sl.qs[nt] = ld16(wrow[nt] + (size_t)blk * 144 + 16 + 32 * g + 16 * h);
        for (int half = 0; half < 2; half++)
            for (int mt = 0; mt < 2; mt++)
                sl.aop[half][mt] = *reinterpret_cast<const u32x4 *>(
                    q8t + ((size_t)(2 * G + half) * mpad + mtok[mt]) * 32 + 16 * h);
        for (int mt = 0; mt < 2; mt++) sl.pv[mt] = P[(size_t)(2 * G + h) * mpad + mtok[mt]];
    };
    for (int nt = 0; nt < NT; nt++) hdr[nt] = ld16(wrow[nt]);
#pragma unroll
    for (int g = 0; g < DIST; g++) fill(slot[g], g);

    for (uint32_t blk = 0; blk < nblk; blk++) {
        const uint32_t nxt = min(blk + 1, nblk - 1);  // last trip: harmless re-read
        u32x4 hd[NT];
        for (int nt = 0; nt < NT; nt++) {
            hd[nt] = hdr[nt];
            hdr[nt] = ld16(wrow[nt] + (size_t)nxt * 144);
        }
#pragma unroll
        for (int g = 0; g < 4; g++) {
            Slot &sl = slot[g % DIST];
            v4i blo[NT], bhi[NT];
            for (int nt = 0; nt < NT; nt++)
                for (int i = 0; i < 4; i++) {
                    blo[nt][i] = (int)(sl.qs[nt][i] & 0x0F0F0F0Fu);
                    bhi[nt][i] = (int)((sl.qs[nt][i] >> 4) & 0x0F0F0F0Fu);
                }
            v4i aop[2][2];
            for (int half = 0; half < 2; half++)
                for (int mt = 0; mt < 2; mt++)
                    for (int i = 0; i < 4; i++) aop[half][mt][i] = (int)sl.aop[half][mt][i];
            const float pv[2] = {sl.pv[0], sl.pv[1]};
            fill(sl, blk * 4 + g + DIST);  // slot consumed: refill it DIST groups ahead
            // scales of sub-blocks 2g, 2g+1 for the lane's weight rows (decode_scales_mins,
            // reference/q4_k.rs:27-49)
            float dsc[NT][2], nc2[NT][2], qneg[NT][2];
            for (int nt = 0; nt < NT; nt++) {
                const float d = h2f(hd[nt][0] & 0xFFFF), dmin = h2f(hd[nt][0] >> 16);
#pragma unroll
                for (int half = 0; half < 2; half++) {
                    const int s = 2 * g + half;
                    uint32_t sc, mn;
                    if (s < 4) {
                        sc = (hd[nt][1] >> (8 * s)) & 63;
                        mn = (hd[nt][2] >> (8 * s)) & 63;
                    } else {
                        sc = ((hd[nt][3] >> (8 * (s - 4))) & 15) | (((hd[nt][1] >> (8 * (s - 4) + 6)) & 3) << 4);
                        mn = ((hd[nt][3] >> (8 * (s - 4) + 4)) & 15) | (((hd[nt][2] >> (8 * (s - 4) + 6)) & 3) << 4);
                    }
                    dsc[nt][half] = d * (float)sc;               // reference/q4_k.rs:280, exact
                    nc2[nt][half] = -(MAGIC_F * dsc[nt][half]);  // exact
                    qneg[nt][half] = -(dmin * (float)mn);        // reference/q4_k.rs:281, exact
                }
            }
#pragma unroll
            for (int half = 0; half < 2; half++) {
                const uint32_t j = blk * 8 + 2 * g + half;
                v16i dres[2][NT];
                for (int mt = 0; mt < 2; mt++)
                    for (int nt = 0; nt < NT; nt++)
                        dres[mt][nt] = __builtin_amdgcn_mfma_i32_32x32x32_i8(aop[half][mt], half ? bhi[nt] : blo[nt], magic, 0, 0, 0);
                for (int mt = 0; mt < 2; mt++) {
                    const u32x4 *dp = reinterpret_cast<const u32x4 *>(&lds_da[((j * 4 + wm * 2 + mt) * 2 + h) * 16]);
                    const u32x4 dav[2] = {dp[0], dp[1]};
                    for (int nt = 0; nt < NT; nt++) {
#pragma unroll
                        for (int i = 0; i < 16; i++) {
                            const uint32_t dbits = (uint32_t)dres[mt][nt][i];
                            // fl(dsc * I), then += * da  (da is an f16 value, exact in fp32)
                            const float t = fmaf(__builtin_bit_cast(float, dbits), dsc[nt][half], nc2[nt][half]);
                            const uint32_t pair = dav[i >> 3][(i >> 1) & 3];
                            const float da = h2f((i & 1) ? (pair >> 16) : (pair & 0xFFFF));
                            acc[mt][nt][i] = fmaf(t, da, acc[mt][nt][i]);
                            if (DUMP) {
                                const uint32_t row = m_wave + mt * 32 + 8 * (i >> 2) + 4 * h + (i & 3);
                                if (row < m && nrow[nt] < n)
                                    sums[((size_t)row * n + nrow[nt]) * nsb + j] = (int)(dbits - MAGIC_BITS);
                            }
                        }
                    }
                }
            }
            // min term of sub-blocks 2g (lanes h = 0) and 2g+1 (lanes h = 1)
            for (int mt = 0; mt < 2; mt++)
                for (int nt = 0; nt < NT; nt++) {
                    const float qv = h ? qneg[nt][1] : qneg[nt][0];
                    acc2[mt][nt] = __builtin_amdgcn_mfma_f32_32x32x2f32(pv[mt], qv, acc2[mt][nt], 0, 0, 0);
                }
        }
    }

    for (int mt = 0; mt < 2; mt++)
        for (int nt = 0; nt < NT; nt++) {
            if (nrow[nt] >= n) continue;
#pragma unroll
            for (int i = 0; i < 16; i++) {
                const uint32_t row = m_wave + mt * 32 + 8 * (i >> 2) + 4 * h + (i & 3);
                if (row < m) {
                    float *o = out + (size_t)row * n + nrow[nt];
                    const float y = acc[mt][nt][i] + acc2[mt][nt][i];
                    *o = accumulate ? *o + y : y;
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

template <int NT, int DIST>
static hipError_t launch_tile_variant(const GemmArgs &a, const uint8_t *q8t, const float *P, const uint16_t *da16,
                                      uint32_t mpad, size_t lds, hipStream_t stream) {
    const dim3 grid(mpad / 128, (a.n + 64 * NT - 1) / (64 * NT));
    hipError_t e = hipSuccess;
    if (lds > 64 * 1024) {  // beyond the default dynamic LDS limit: opt in (up to the 160 KB of a CU)
        e = a.sums ? hipFuncSetAttribute(reinterpret_cast<const void *>(&gemm_q4k_q8_kernel<NT, DIST, true>),
                                         hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds)
                   : hipFuncSetAttribute(reinterpret_cast<const void *>(&gemm_q4k_q8_kernel<NT, DIST, false>),
                                         hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (e != hipSuccess) return e;
    }
    if (a.sums)
        hipLaunchKernelGGL((gemm_q4k_q8_kernel<NT, DIST, true>), grid, dim3(256), lds, stream, a.W, q8t, P, da16, a.out,
                           a.sums, a.m, mpad, a.n, a.k, a.accumulate);
    else
        hipLaunchKernelGGL((gemm_q4k_q8_kernel<NT, DIST, false>), grid, dim3(256), lds, stream, a.W, q8t, P, da16, a.out,
                           a.sums, a.m, mpad, a.n, a.k, a.accumulate);
    return hipGetLastError();
}

static hipError_t launch_tiles(const GemmArgs &a, const uint8_t *q8t, const float *P, const uint16_t *da16,
                               uint32_t mpad, size_t lds, hipStream_t stream) {
    switch (g_gemm_variant) {
    case 1: return launch_tile_variant<1, 1>(a, q8t, P, da16, mpad, lds, stream);
    case 2: return launch_tile_variant<1, 2>(a, q8t, P, da16, mpad, lds, stream);
    case 3: return launch_tile_variant<1, 4>(a, q8t, P, da16, mpad, lds, stream);
    case 4: return launch_tile_variant<2, 1>(a, q8t, P, da16, mpad, lds, stream);
    case 5: return launch_tile_variant<2, 2>(a, q8t, P, da16, mpad, lds, stream);
    case 6: return launch_tile_variant<2, 4>(a, q8t, P, da16, mpad, lds, stream);
    default: return launch_tile_variant<1, 2>(a, q8t, P, da16, mpad, lds, stream);
    }
}

bool gemm_uses_tiles(uint32_t type, uint32_t m, uint32_t k) {
    // LDS holds the f16 token scales of 128 tokens for the whole k: k/32 * 256 bytes
    return type == OXQ_TYPE_Q4_K && m >= 8 && (size_t)(k / 32) * 256 <= 160 * 1024;
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
    const size_t lds = (size_t)nsb * 256;
    return launch_tiles(a, q8t, P, da16, mpad, lds, stream);
}

}  // namespace oxq
