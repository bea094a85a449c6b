// The streamed form of the int8-MFMA tile kernel (oxq_gemm_tile.hpp): same arithmetic, same operand
// layouts, the same exact integer sums -- a different way of bringing the weights in.
//
//   out[m x n] (+)= A_q8[m rows of Q8_0 blocks] x W[n x k]^T
// (the reference's gemm loop over matvec_q8_fused, crates/oxillama-quant/src/reference/q4_k.rs:186-201,
// :218-333), for the formats whose blocks are a whole number of 16-byte pieces (Q4_K, IQ4_XS).
//
// Raw weight blocks go from global memory to LDS with 16-byte loads that write LDS directly (no
// registers): consecutive lanes take consecutive 16-byte pieces of a row's k-run, so one load
// instruction covers 1 KB in at most 16 cache lines where the tile kernel's lane-per-row loads touch
// 32-64.  Consumers read their B operands (raw nibbles) from a ring of LDS slots with ds_read_b128 and
// unpack them in registers; token bytes, scale factors and the two-VALU-operations-per-result stage are
// the tile kernel's.  Work groups are persistent: each walks a strided list of tiles and the weight
// stream runs across tile boundaries.  One s_barrier per stage hands a slot over.  Two forms:
//  * many tokens (four waves, two work groups per compute unit): every wave requests its share of the
//    stage after next right behind the barrier; a wave owns MT x NT MFMA tiles of 32 tokens x 32 rows.
//  * few tokens (four consumer waves and a producer wave): the producer does nothing but request weight
//    bytes, NSTAGE - 1 stages ahead; its loads are the only entries of its memory counter, so the weight
//    stream from HBM is not coupled to the consumers' short-latency token loads (one wave's loads retire
//    in order).  The four consumers share one tile and each walk a quarter of k; the partial tiles meet
//    in LDS in a fixed order.
// A consumer's stage is written out as a software pipeline (requests a tile-step ahead, the MFMA of
// tile-step ts + 2 before the VALU work of ts + 1, also across groups) and pinned with scheduling barriers.
//
// Measured on MI355X (Q4_K, 512 x 14336 x 4096): the memory path does what it was built for -- texture
// unit busy 28 % of the run instead of 51 %, 13.6 cache-line accesses per load instead of 21, L1 misses
// halved -- and the kernel is no faster (143 us against 126 us): with two waves per SIMD the VALU stage,
// the LDS reads of the token scales and the matrix core do not overlap well enough, whichever way the
// weights arrive.  The tile kernel therefore stays the default; this one is selected with
// oxq_set_gemm_variant(100 and up) and is held to the same parity tests.
#pragma once
#include "oxq_gemm_tile.hpp"

namespace oxq {

#define OXQ_LDS_PTR(p) ((__attribute__((address_space(3))) void *)(p))

struct __attribute__((aligned(8))) LdsU4A8 {
    uint32_t v[4];
};
__device__ __forceinline__ u32x4 lds16(const uint8_t *p) { return *reinterpret_cast<const u32x4 *>(p); }
__device__ __forceinline__ u32x4 lds16_a8(const uint8_t *p) {  // 16 bytes at an 8-byte-aligned LDS address
    const LdsU4A8 t = *reinterpret_cast<const LdsU4A8 *>(p);
    return u32x4{t.v[0], t.v[1], t.v[2], t.v[3]};
}

// What a format needs to be streamed: S super-blocks of a row per stage (SEG bytes, a multiple
// of 16 and 16-byte aligned in global memory for every stage), and how a lane picks its bytes out of
// the staged run of its row.
template <class F>
struct Stream {
    static constexpr bool OK = false;
};
template <>
struct Stream<TileQ4K> {
    static constexpr bool OK = true, PREFILL = true;
    static constexpr int S = 1;
    static constexpr uint32_t SEG = 144;
    static __device__ __forceinline__ void fetch(const uint8_t *row, uint32_t b, uint32_t h, uint32_t g, u32x4 (&qs)[1]) {
        qs[0] = lds16(row + 144 * b + 16 + 32 * g + 16 * h);
    }
    static __device__ __forceinline__ void load_hdr(const uint8_t *row, uint32_t b, TileQ4K::Hdr &hd) {
        hd.w = lds16(row + 144 * b);
    }
};
template <>
struct Stream<TileIQ4XS> {
    // PREFILL false: with two super-blocks per stage the unrolled stage of a two-tile wave does not fit the
    // register file; many-token shapes of this format stay on the tile kernel
    static constexpr bool OK = true, PREFILL = false;
    static constexpr int S = 2;  // 136-byte blocks: pairs of them start on 16-byte boundaries
    static constexpr uint32_t SEG = 272;
    static __device__ __forceinline__ void fetch(const uint8_t *row, uint32_t b, uint32_t h, uint32_t g, u32x4 (&qs)[1]) {
        qs[0] = lds16_a8(row + 136 * b + 8 + 32 * g + 16 * h);
    }
    static __device__ __forceinline__ void load_hdr(const uint8_t *row, uint32_t b, TileIQ4XS::Hdr &hd) {
        hd.w = lds16_a8(row + 136 * b);
    }
};

// s_waitcnt vmcnt(n), other counters untouched (gfx9 encoding: vmcnt = imm[15:14]:imm[3:0]).
template <int N>
__device__ __forceinline__ void wait_vmcnt() {
    static_assert(N >= 0 && N <= 63, "vmcnt is six bits");
    __builtin_amdgcn_s_waitcnt((N & 15) | ((N >> 4) << 14) | (7 << 4) | (15 << 8));
}
// Work-group barrier that the compiler may not move memory operations across, without the
// memory-counter drain of __syncthreads (the consumers keep their token loads in flight across it).
__device__ __forceinline__ void stage_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

// One tile of the walk: which tokens, which weight rows, which matrix.
struct StreamTile {
    bool live;
    uint32_t expert, m_wg, n_wg, row_end;
};

template <class F, int MT, int NT, int WM, int NSTAGE, bool PRODUCER, bool DUMP, int ADIST>
__device__ __forceinline__ void gemm_stream_body(
    const uint8_t *__restrict__ W, const uint8_t *__restrict__ q8t, const float *__restrict__ P,
    const uint16_t *__restrict__ da16, float *__restrict__ out, int32_t *__restrict__ sums, uint32_t m, uint32_t mpad,
    uint32_t n, uint32_t k, int accumulate, const float *__restrict__ bias, uint32_t m_tiles, uint32_t n_tiles,
    const int32_t *__restrict__ offsets, size_t w_stride, uint32_t n_items, uint32_t n_experts) {
    using SF = Stream<F>;
    constexpr bool SPLITK = WM == 0;  // the four consumers share one tile and each walk a quarter of k
    constexpr int WMX = SPLITK ? 1 : WM, WN = SPLITK ? 1 : 4 / WMX;
    constexpr int WG_TOK = 32 * MT * WMX, WG_ROWS = 32 * NT * WN, MTILES = MT * WMX;
    constexpr int S = SF::S;
    constexpr uint32_t SEG = SF::SEG;
    constexpr int W_ROWS = 32 * NT;                 // weight rows of one consumer
    constexpr int PPR = SEG / 16;                   // 16-byte pieces of one row per stage
    constexpr int PIECES = W_ROWS * PPR, NL = (PIECES + 63) / 64;  // loads per row set and stage
    constexpr int SLOT = NL * 1024;
    constexpr int NSETS = SPLITK ? 4 : WN;          // row sets (each with its own k position) per stage
    constexpr int LPS = NL * NSETS;                 // loads per stage
    constexpr int NP = 2 + (F::HAS_MIN ? 1 : 0);
    constexpr int LPR = 64 / W_ROWS, SPL = 8 / LPR;  // scale decode: lanes per row, sub-blocks per lane
    constexpr int ISSUERS = PRODUCER ? 1 : 4;       // waves that request weight bytes
    constexpr int SHARE = (LPS + ISSUERS - 1) / ISSUERS;  // loads per stage and requesting wave
    // stages the producer wave lets be outstanding behind the one it waits for: the ring allows NSTAGE - 2, the
    // six bits of the memory counter 63 / LPS
    constexpr int BEHIND = (NSTAGE - 2) * LPS <= 63 ? NSTAGE - 2 : 63 / LPS;
    // the zero-point term in accumulators of its own (a wave with one tile has nothing else to hide the fp32
    // MFMA's latency behind), or added into the main ones as the tile kernel does (registers are scarcer)
    constexpr bool SPLIT_MIN = F::HAS_MIN && MT * NT == 1;
    static_assert(F::KSPLIT == 1 && tile_min_planes<F>::value == 1 && F::NQ == 1, "streamed formats have 32-weight groups");
    static_assert(NT <= 2 && NSTAGE >= 2 && (PRODUCER || NSTAGE == 2), "ring configuration");
    static_assert(SEG % 16 == 0 && SEG == S * F::BLOCK_BYTES, "stage geometry");

    // Ring slots are separate arrays: where the waves that read a slot also request the next one (no producer
    // wave), the compiler's memory-counter tracking can then tell a read of one slot from a request into another.
    __shared__ __align__(16) uint8_t ring_a[NSETS][SLOT];
    __shared__ __align__(16) uint8_t ring_b[NSETS][SLOT];
    __shared__ __align__(16) uint8_t ring_c[NSTAGE > 2 ? NSETS : 1][NSTAGE > 2 ? SLOT : 16];
    __shared__ __align__(16) uint8_t ring_d[NSTAGE > 3 ? NSETS : 1][NSTAGE > 3 ? SLOT : 16];
    __shared__ float lds_sc[4][S][8][NP][W_ROWS];
    __shared__ float lds_red[SPLITK ? 4 : 1][SPLITK ? MT * NT : 1][SPLITK ? 16 : 1][SPLITK ? 64 : 1];
    extern __shared__ uint16_t lds_da[];  // [nsb][MTILES][2 halves][16] f16 token scales of the current token tile
    static_assert(NSTAGE <= 4, "four ring slots are declared");
    auto ring_slot = [&](uint32_t slot, uint32_t set_) -> uint8_t * {
        return slot == 0 ? &ring_a[set_][0] : slot == 1 ? &ring_b[set_][0] : slot == 2 ? &ring_c[set_][0] : &ring_d[set_][0];
    };

    const uint32_t nsb = k / 32, nblk = k / 256, nst = nblk / S;
    const uint32_t tid = threadIdx.x, lane = tid & 63;
    const uint32_t wave = (uint32_t)__builtin_amdgcn_readfirstlane((int)(tid >> 6));
    const bool producer = PRODUCER && wave == 4;
    const uint32_t c = lane & 31, h = lane >> 5;
    const uint32_t wm = SPLITK ? 0 : (wave & 3) % WMX, wn = SPLITK ? 0 : (wave & 3) / WMX;
    const uint32_t set = SPLITK ? (wave & 3) : wn;  // the ring's row set this consumer reads
    // stages of one consumer per tile, and where its k range starts
    const uint32_t nst_w = SPLITK ? nst / 4 : nst;
    const uint32_t st0 = SPLITK ? (wave & 3) * nst_w : 0;
    const uint32_t row_bytes = nblk * F::BLOCK_BYTES;
    const uint32_t n_groups = (n_tiles + 7) / 8;

    // item -> tile.  Items are dealt round-robin to the 8 XCDs (work-group ids are); inside an XCD the token
    // tiles of one set of weight rows are neighbours, so their weight reads meet in that XCD's L2.  Grouped
    // form: token tiles outermost per expert, so the tiles past an expert's rows form one run.
    auto tile_of = [&](uint32_t item) {
        StreamTile t;
        const uint32_t per_expert = 8 * n_groups * m_tiles;
        t.expert = item / per_expert;
        const uint32_t it = item % per_expert;
        const uint32_t xcd = it & 7, loc = it >> 3;
        uint32_t n_tile, m_tile, row0 = 0;
        t.row_end = m;
        if (offsets) {
            m_tile = loc / n_groups;
            n_tile = (loc % n_groups) * 8 + xcd;
            row0 = (uint32_t)offsets[t.expert];
            t.row_end = (uint32_t)offsets[t.expert + 1];
        } else {
            n_tile = (loc / m_tiles) * 8 + xcd;
            m_tile = loc % m_tiles;
        }
        t.m_wg = row0 + m_tile * WG_TOK;
        t.n_wg = n_tile * WG_ROWS;
        t.live = n_tile < n_tiles && t.m_wg < t.row_end;
        return t;
    };

    // ---------------- the weight stream: an issue cursor that runs ahead of the walk ----------------
    uint32_t p_item = blockIdx.x, p_stage = 0;  // next stage to request: stage p_stage of the tile of item p_item
    uint32_t p_issued = 0;                      // stages requested so far
    uint32_t prow[SHARE], pcol[SHARE], pset[SHARE], pdst[SHARE];  // the lane's piece of each load of this wave
    bool pvalid[SHARE];
#pragma unroll
    for (int i = 0; i < SHARE; i++) {
        const uint32_t ld = PRODUCER ? (uint32_t)i : (uint32_t)i * 4 + (wave & 3);  // load index within the stage
        pvalid[i] = ld < (uint32_t)LPS;
        const uint32_t ldc = min(ld, (uint32_t)LPS - 1);
        const uint32_t j = ldc % NL;
        pset[i] = ldc / NL;
        pdst[i] = j * 1024;
        const uint32_t piece = min(64 * j + lane, (uint32_t)(PIECES - 1));  // past the end: repeat the last piece
        prow[i] = piece / PPR;
        pcol[i] = (piece % PPR) * 16;
    }
    // Request this wave's share of the next stage of the stream into ring slot `slot`, if there is one.
    auto issue_next = [&](uint32_t slot) -> bool {
        StreamTile t;
        while (true) {
            if (p_item >= n_items) return false;
            t = tile_of(p_item);
            if (t.live) break;
            p_item += gridDim.x;
        }
        const uint8_t *Wt = W + (size_t)t.expert * w_stride;
        const __amdgpu_buffer_rsrc_t rs = __builtin_amdgcn_make_buffer_rsrc(
            const_cast<uint8_t *>(Wt), 0, (int)min((size_t)n * row_bytes, (size_t)0xFFFFFFF0u), BUFFER_FLAGS);
#pragma unroll
        for (int i = 0; i < SHARE; i++) {
            if (!pvalid[i]) continue;  // wave-uniform
            // row set s: rows n_wg + s * W_ROWS .. (prefill), or the tile's rows at k quarter s (split k)
            const uint32_t rbase = t.n_wg + (SPLITK ? 0 : pset[i] * W_ROWS);
            const uint32_t stage = (SPLITK ? pset[i] * nst_w : 0) + p_stage;
            const uint32_t row = min(rbase + prow[i], n - 1);  // rows past n: re-read the last one (never used)
            __builtin_amdgcn_raw_ptr_buffer_load_lds(rs, OXQ_LDS_PTR(ring_slot(slot, pset[i]) + pdst[i]), 16,
                                                     row * row_bytes + pcol[i], stage * SEG, 0, 0);
        }
        p_issued++;
        if (++p_stage == nst_w) {
            p_stage = 0;
            p_item += gridDim.x;
        }
        return true;
    };
    bool p_more = true;  // the stream has stages left to request
    if (producer) {
#pragma unroll
        for (int i = 0; i < NSTAGE - 1; i++)
            if (p_more) p_more = issue_next(i);
    }
    if constexpr (!PRODUCER) p_more = issue_next(0);

    // ---------------- consumer state ----------------
    v16i magic;
    for (int i = 0; i < 16; i++) magic[i] = (int)MAGIC_BITS;
    const __amdgpu_buffer_rsrc_t rs_a =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<uint8_t *>(q8t), 0, (int)(nsb * mpad * 32), BUFFER_FLAGS);
    const __amdgpu_buffer_rsrc_t rs_p =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<float *>(P), 0, (int)(nsb * mpad * 4), BUFFER_FLAGS);
    const uint32_t drow = lane % W_ROWS, ds0 = SPL * (lane / W_ROWS);

    uint32_t consumed = 0;             // stages consumed so far by this work group
    uint32_t staged_m = 0xFFFFFFFFu;   // token tile whose scales lds_da holds

    for (uint32_t item = blockIdx.x; item < n_items; item += gridDim.x) {
        const StreamTile t = tile_of(item);
        if (!t.live) continue;  // the same decision in every wave
        const uint32_t row_end = t.row_end;
        const uint32_t m_wave = t.m_wg + wm * (32 * MT), n_wave = t.n_wg + wn * (32 * NT);

        // Token scales of this tile's tokens into LDS (permuted so that the 16 values a lane needs for
        // one MFMA tile are 32 contiguous bytes), unless the previous tile had the same tokens.
        if (t.m_wg != staged_m) {
            stage_barrier();  // every consumer is done reading the previous tile's scales
            if (!producer) {
                constexpr uint32_t CH = WG_TOK / 8;  // 8-token chunks per sub-block
                const uint32_t n_tasks = nsb * CH;
                for (uint32_t base = 0; base < n_tasks; base += 4 * 256) {
                    u32x4 v[4];
#pragma unroll
                    for (int q = 0; q < 4; q++) {
                        const uint32_t task = min(base + q * 256 + (tid & 255), n_tasks - 1);
                        const uint32_t j = task / CH, ch = task % CH;
                        v[q] = ld16(reinterpret_cast<const uint8_t *>(da16 + (size_t)j * mpad + t.m_wg + 8 * ch));
                    }
#pragma unroll
                    for (int q = 0; q < 4; q++) {
                        const uint32_t task = base + q * 256 + (tid & 255);
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
            staged_m = t.m_wg;
            stage_barrier();
        }

        // acc: the scaled group sums; accm: the zero-point term, kept apart so that its fp32 MFMAs and the
        // VALU work on acc never wait for each other; added once at the end of the tile.
        v16f acc[MT][NT], accm[SPLIT_MIN ? MT : 1][SPLIT_MIN ? NT : 1];
        for (int a = 0; a < MT; a++)
            for (int b = 0; b < NT; b++)
                for (int i = 0; i < 16; i++) acc[a][b][i] = 0.0f;
        if constexpr (SPLIT_MIN)
            for (int i = 0; i < 16; i++) accm[0][0][i] = 0.0f;
        uint32_t nrow[NT];
        for (int nt = 0; nt < NT; nt++) nrow[nt] = n_wave + nt * 32 + c;
        uint32_t aq_off[MT], pq_off[MT];
        for (int mt = 0; mt < MT; mt++) {
            const uint32_t tok = m_wave + mt * 32 + c;  // always < mpad
            aq_off[mt] = tok * 32 + 16 * h;             // the lane's 16 bytes of its token's activation block
            pq_off[mt] = (h * mpad + tok) * 4;          // P of the sub-block the lane's half feeds to the min term
        }
        struct Ops {
            u32x4 a[2][MT];
            float pv[MT];
        };
        Ops ops[4];  // token bytes: ring of four slots (slot = group % 4), requested ADIST groups ahead
        static_assert(ADIST >= 1 && ADIST <= 3, "token prefetch distance");
        const uint32_t g_first = st0 * S * 4, g_last = (st0 + nst_w) * S * 4 - 1;  // this consumer's groups (4 per block)
        auto fetch_a = [&](Ops &o, uint32_t G) {
            G = min(G, g_last);  // past the end: re-read the last group (result unused)
            const uint32_t blk8 = (G >> 2) * 8, g = G & 3;
            for (int e = 0; e < 2; e++)
                for (int mt = 0; mt < MT; mt++)
                    o.a[e][mt] = buf16(rs_a, aq_off[mt], (blk8 + F::sub_block(g, e)) * mpad * 32);
            if (F::HAS_MIN)
                for (int mt = 0; mt < MT; mt++)
                    o.pv[mt] = __builtin_bit_cast(
                        float, __builtin_amdgcn_raw_buffer_load_b32(rs_p, pq_off[mt], (blk8 + F::sub_block(g, 0)) * mpad * 4, 0));
        };
        if (!producer) {
#pragma unroll
            for (int d = 0; d < ADIST; d++) fetch_a(ops[d], g_first + d);
        }

        // One stage of this consumer: S blocks x 4 groups x T tiles, as one software pipeline.  The int8 MFMA of
        // tile-step ts + 2 is issued before the VALU work of tile-step ts + 1, also across group boundaries; the
        // B operands of group gi + 1 are read from the ring at the start of group gi and unpacked in its shadow.
        auto consume_stage = [&](const uint8_t *slot, uint32_t blk0) {
            constexpr int T = 2 * MT * NT, NG = 4 * S, NTS = NG * T;
            const uint32_t wv = wave & 3;
            // the blocks' scale factors, decoded once per wave into its own table
#pragma unroll
            for (int b = 0; b < S; b++) {
                typename F::Hdr hd;
                SF::load_hdr(slot + drow * SEG, b, hd);
#pragma unroll
                for (int e = 0; e < SPL; e++) {
                    const uint32_t s = ds0 + e;
                    float dsc[1], qneg;
                    F::factors(hd, e, s, dsc, qneg);
                    lds_sc[wv][b][s][0][drow] = dsc[0];
                    lds_sc[wv][b][s][1][drow] = -(MAGIC_F * dsc[0]);  // exact
                    if constexpr (F::HAS_MIN) lds_sc[wv][b][s][NP - 1][drow] = qneg;
                }
            }
            u32x4 raw[NT][1];
            BOperand<1> bop[2][NT][2];
            auto fetch_b = [&](int gi) {
                for (int nt = 0; nt < NT; nt++) SF::fetch(slot + (nt * 32 + c) * SEG, gi / 4, h, gi % 4, raw[nt]);
            };
            auto unpack_b = [&](int gi) {
                for (int nt = 0; nt < NT; nt++) F::operands(raw[nt], gi % 4, bop[gi & 1][nt]);
            };
            auto mfma_ts = [&](int ts) {
                const int gi = ts / T, tt = ts % T;
                const int e = tt / (MT * NT), mt = (tt / NT) % MT, nt = tt % NT;
                v4i aop;
                for (int i = 0; i < 4; i++) aop[i] = (int)ops[gi % 4].a[e][mt][i];
                return __builtin_amdgcn_mfma_i32_32x32x32_i8(aop, bop[gi & 1][nt][e].k32, magic, 0, 0, 0);
            };
            // the scale operands of a tile-step: the weight rows' two factors, the 16 tokens' f16 scales
            struct Sc {
                float dsc, nc2;
                u32x4 dav[2];
            };
            auto load_sc = [&](int ts, Sc &sc) {
                const int gi = ts / T, tt = ts % T;
                const int b = gi / 4, g = gi % 4;
                const int e = tt / (MT * NT), mt = (tt / NT) % MT, nt = tt % NT;
                const uint32_t s = F::sub_block(g, e), j = (blk0 + b) * 8 + s;
                sc.dsc = lds_sc[wv][b][s][0][nt * 32 + c];
                sc.nc2 = lds_sc[wv][b][s][1][nt * 32 + c];
                const u32x4 *dp = reinterpret_cast<const u32x4 *>(&lds_da[((j * MTILES + wm * MT + mt) * 2 + h) * 16]);
                sc.dav[0] = dp[0];
                sc.dav[1] = dp[1];
            };
            fetch_b(0);
            unpack_b(0);
            v16i dq[2];
            dq[0] = mfma_ts(0);
            dq[1] = mfma_ts(1);
            Sc scs[2];
            load_sc(0, scs[0]);
            float qv[NT];  // zero-point factors of the current group's two sub-blocks (lanes h = 0: the first, h = 1: the second)
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int ts = 0; ts < NTS; ts++) {
                const int gi = ts / T, tt = ts % T;
                const int b = gi / 4, g = gi % 4;
                const int e = tt / (MT * NT), mt = (tt / NT) % MT, nt = tt % NT;
                const uint32_t blk = blk0 + b;
                // requests first: token bytes ADIST groups ahead, the next group's weight bytes, the next tile-step's scales
                if (tt == 0) {
                    fetch_a(ops[(gi + ADIST) % 4], blk0 * 4 + gi + ADIST);
                    if (gi + 1 < NG) fetch_b(gi + 1);
                    if constexpr (F::HAS_MIN)
                        for (int nt2 = 0; nt2 < NT; nt2++) qv[nt2] = lds_sc[wv][b][F::sub_block(g, 0) + h][NP - 1][nt2 * 32 + c];
                }
                if (ts + 1 < NTS) load_sc(ts + 1, scs[(ts + 1) & 1]);
                __builtin_amdgcn_sched_barrier(0);  // the requests stay up here, a whole tile-step ahead of their use
                const Sc &sc = scs[ts & 1];
                const uint32_t j = blk * 8 + F::sub_block(g, e);
                const v16i dres = dq[ts & 1];
#pragma unroll
                for (int i = 0; i < 16; i++) {
                    const uint32_t dbits = (uint32_t)dres[i];
                    const float x = fmaf(__builtin_bit_cast(float, dbits), sc.dsc, sc.nc2);  // fl(dsc * I)
                    const uint32_t pair = sc.dav[i >> 3][(i >> 1) & 3];
                    const float da = h2f((i & 1) ? (pair >> 16) : (pair & 0xFFFF));
                    acc[mt][nt][i] = fmaf(x, da, acc[mt][nt][i]);
                    if (DUMP) {
                        const uint32_t row = m_wave + mt * 32 + 8 * (i >> 2) + 4 * h + (i & 3);
                        if (row < row_end && nrow[nt] < n)
                            sums[((size_t)row * n + nrow[nt]) * nsb + j] = (int)(dbits - MAGIC_BITS);
                    }
                }
                if (tt == T - 2 && gi + 1 < NG) unpack_b(gi + 1);
                if (ts + 2 < NTS) dq[ts & 1] = mfma_ts(ts + 2);
                if constexpr (F::HAS_MIN) {
                    // zero-point term of the group (both sub-blocks in one K = 2 MFMA), right behind the tile's first
                    // VALU pass: the accumulators are next touched MT * NT tile-steps later
                    if (e == 0) {
                        if constexpr (SPLIT_MIN)
                            accm[mt][nt] = __builtin_amdgcn_mfma_f32_32x32x2f32(ops[gi % 4].pv[mt], qv[nt], accm[mt][nt], 0, 0, 0);
                        else
                            acc[mt][nt] = __builtin_amdgcn_mfma_f32_32x32x2f32(ops[gi % 4].pv[mt], qv[nt], acc[mt][nt], 0, 0, 0);
                    }
                }
                __builtin_amdgcn_sched_barrier(0);  // tile-steps stay in this order: the pipeline is written out above
            }
        };

        // ---- the stages of this tile: one barrier each ----
        if constexpr (PRODUCER) {
            for (uint32_t x = 0; x < nst_w; x++) {
                if (producer) {
                    // stage `consumed` has landed when at most BEHIND stages requested after it are outstanding
                    if (p_issued - consumed >= (uint32_t)(BEHIND + 1))
                        wait_vmcnt<BEHIND * LPS>();
                    else
                        wait_vmcnt<0>();  // the stream is ending: fewer are behind it
                }
                stage_barrier();
                if (producer) {
                    if (p_more) p_more = issue_next(p_issued % NSTAGE);  // into the slot the consumers have just left
                } else {
                    consume_stage(ring_slot(consumed % NSTAGE, set), (st0 + x) * S);
                }
                consumed++;
            }
        } else {
            // no producer wave: every wave requests its share of the stage after next right behind the barrier
            // (two slots, stage parity = slot: the caller guarantees an even number of stages per tile)
            for (uint32_t x = 0; x < nst_w; x += 2) {
                wait_vmcnt<0>();  // this wave's share of the stage in ring_a (and its token bytes in flight)
                stage_barrier();
                if (p_more) p_more = issue_next(1);
                consume_stage(&ring_a[set][0], (st0 + x) * S);
                wait_vmcnt<0>();
                stage_barrier();
                if (p_more) p_more = issue_next(0);
                consume_stage(&ring_b[set][0], (st0 + x + 1) * S);
            }
            consumed += nst_w;
        }
        if constexpr (SPLIT_MIN) {
            for (int i = 0; i < 16; i++) acc[0][0][i] += accm[0][0][i];
        }

        // ---- results ----
        if constexpr (SPLITK) {
            // The four partial tiles meet in LDS; consumer w then adds registers 4w..4w+3 of every tile in the
            // fixed order (w0 + w1) + (w2 + w3) and stores them.
            if (!producer) {
                for (int mt = 0; mt < MT; mt++)
                    for (int nt = 0; nt < NT; nt++)
#pragma unroll
                        for (int i = 0; i < 16; i++) lds_red[wave & 3][mt * NT + nt][i][lane] = acc[mt][nt][i];
            }
            stage_barrier();  // the next write to lds_red comes after at least one more stage barrier
            if (!producer) {
                for (int mt = 0; mt < MT; mt++)
                    for (int nt = 0; nt < NT; nt++) {
                        if (nrow[nt] >= n) continue;
#pragma unroll
                        for (int ii = 0; ii < 4; ii++) {
                            const uint32_t i = 4 * (wave & 3) + ii;
                            const uint32_t row = m_wave + mt * 32 + 8 * (wave & 3) + 4 * h + ii;
                            if (row < row_end) {
                                const int tl = mt * NT + nt;
                                const float y = (lds_red[0][tl][i][lane] + lds_red[1][tl][i][lane]) +
                                                (lds_red[2][tl][i][lane] + lds_red[3][tl][i][lane]);
                                float *o = out + (size_t)row * n + nrow[nt];
                                *o = accumulate ? *o + y : bias ? y + bias[nrow[nt]] : y;
                            }
                        }
                    }
            }
        } else if (!producer) {
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
    }
}

// The kernel proper.  With a producer wave (few tokens: the weight stream from HBM paces the kernel) a work group is
// five waves and one of them per compute unit runs, two waves on one SIMD at most; without (prefill: the VALU
// paces the kernel) it is four waves, two work groups per compute unit, two waves per SIMD.  Either way the
// register budget is that of two waves per SIMD.
template <class F, int MT, int NT, int WM, int NSTAGE, bool PRODUCER, bool DUMP, int ADIST>
__global__ __launch_bounds__(PRODUCER ? 320 : 256) __attribute__((amdgpu_waves_per_eu(2, 2))) void gemm_stream_kernel(
    const uint8_t *__restrict__ W, const uint8_t *__restrict__ q8t, const float *__restrict__ P,
    const uint16_t *__restrict__ da16, float *__restrict__ out, int32_t *__restrict__ sums, uint32_t m, uint32_t mpad,
    uint32_t n, uint32_t k, int accumulate, const float *__restrict__ bias, uint32_t m_tiles, uint32_t n_tiles,
    const int32_t *__restrict__ offsets, size_t w_stride, uint32_t n_items, uint32_t n_experts) {
    gemm_stream_body<F, MT, NT, WM, NSTAGE, PRODUCER, DUMP, ADIST>(W, q8t, P, da16, out, sums, m, mpad, n, k, accumulate,
                                                                   bias, m_tiles, n_tiles, offsets, w_stride, n_items,
                                                                   n_experts);
}

// True when the streamed kernel takes this shape: whole stages (per consumer in the split-k form; an even
// number of them per tile without a producer wave), 16-byte-aligned rows, offsets that fit the 32-bit lane
// offset of a buffer load.
template <class F>
static bool stream_takes(const GemmArgs &a, bool splitk, bool producer) {
    if constexpr (!Stream<F>::OK) {
        return false;
    } else {
        const uint32_t nblk = a.k / 256;
        const size_t row_bytes = (size_t)nblk * F::BLOCK_BYTES;
        if (a.k % 256 != 0 || nblk % (Stream<F>::S * (splitk ? 4 : 1) * (producer ? 1 : 2)) != 0) return false;
        if (row_bytes % 16 != 0 || (reinterpret_cast<uintptr_t>(a.W) & 15) != 0 || (a.w_stride & 15) != 0) return false;
        return (size_t)a.n * row_bytes < 0xFFFF0000ull;
    }
}

// Static LDS of an instantiation (ring, scale tables, split-k reduction), without the token scales.
template <class F, int MT, int NT, int WM, int NSTAGE>
constexpr size_t stream_static_lds() {
    if constexpr (!Stream<F>::OK) {
        return 0;
    } else {
        constexpr int WMX = WM ? WM : 1;
        constexpr int NL = (32 * NT * (int)(Stream<F>::SEG / 16) + 63) / 64, NSETS = WM ? 4 / WMX : 4;
        return (size_t)NSTAGE * NSETS * NL * 1024 + 4 * Stream<F>::S * 8 * (2 + (F::HAS_MIN ? 1 : 0)) * 32 * NT * 4 +
               (WM ? 4 : 4 * MT * NT * 16 * 64 * 4) + 64;
    }
}

template <class F, int MT, int NT, int WM, int NSTAGE, bool PRODUCER, bool DUMP, int ADIST = 1>
static hipError_t launch_stream(const GemmArgs &a, const TilePlan &p, hipStream_t stream, uint32_t wgs_per_cu) {
    if constexpr (!Stream<F>::OK || stream_static_lds<F, MT, NT, WM, NSTAGE>() > 140 * 1024 || (!PRODUCER && !Stream<F>::PREFILL)) {
        return hipErrorNotSupported;  // not instantiated: the ring would not leave room for the token scales
    } else {
        if (!stream_takes<F>(a, WM == 0, PRODUCER)) return hipErrorNotSupported;
        constexpr int WMX = WM ? WM : 1, WNX = WM ? 4 / WMX : 1;
        constexpr uint32_t WG_TOK = 32 * MT * WMX, WG_ROWS = 32 * NT * WNX;
        const uint32_t rows = a.offsets ? a.max_rows : a.m;
        const uint32_t m_tiles = (rows + WG_TOK - 1) / WG_TOK, n_tiles = (a.n + WG_ROWS - 1) / WG_ROWS;
        const uint32_t n_experts = a.offsets ? a.n_experts : 1;
        const uint32_t n_items = 8 * ((n_tiles + 7) / 8) * m_tiles * n_experts;
        // persistent work groups: a multiple of 8 (one residue class of items per XCD), at most one per item
        uint32_t grid = device_cus() * wgs_per_cu;
        if (grid > n_items) grid = n_items;
        grid = grid / 8 * 8;
        if (grid == 0) grid = 8;
        const size_t lds = (size_t)(a.k / 32) * WG_TOK * 2;
        if (lds + stream_static_lds<F, MT, NT, WM, NSTAGE>() > 160 * 1024) return hipErrorNotSupported;
        auto kern = &gemm_stream_kernel<F, MT, NT, WM, NSTAGE, PRODUCER, DUMP, ADIST>;
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kern),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (e != hipSuccess) return e;
        constexpr uint32_t threads = PRODUCER ? 320 : 256;
        note_launch(PRODUCER ? "gemm_stream_kernel_producer" : "gemm_stream_kernel", F::TYPE, MT, NT, WM, NSTAGE, grid, 1, threads);
        hipLaunchKernelGGL(kern, dim3(grid), dim3(threads), lds, stream, a.W, p.q8t, p.P, p.da16, a.out, a.sums, a.m,
                           p.mpad, a.n, a.k, a.accumulate, a.bias, m_tiles, n_tiles, a.offsets, a.w_stride, n_items,
                           n_experts);
        return hipGetLastError();
    }
}

// Shape choice of the streamed kernel.  hipErrorNotSupported: the caller falls back to the tile kernel.
template <class F>
static hipError_t launch_streamed(const GemmArgs &a, const TilePlan &p, hipStream_t stream, uint32_t rows, int variant) {
    if constexpr (!Stream<F>::OK) {
        return hipErrorNotSupported;
    } else {
        if (a.sums) {  // debug dump: the production shapes with the extra stores
            if (rows > 64) return launch_stream<F, 2, 1, 2, 2, false, true, 2>(a, p, stream, 2);
            if (rows > 32) return hipErrorNotSupported;
            const hipError_t e = launch_stream<F, 1, 1, 0, 3, true, true, 3>(a, p, stream, 1);
            return e != hipErrorNotSupported ? e : launch_stream<F, 1, 1, 0, 2, true, true, 3>(a, p, stream, 1);
        }
        switch (variant) {
        case 101: return launch_stream<F, 2, 1, 2, 2, false, false, 2>(a, p, stream, 2);  // 128 tokens x 64 rows per work group
        case 102: return launch_stream<F, 1, 2, 4, 2, false, false, 2>(a, p, stream, 2);  // 128 tokens x 64 rows, one row set
        case 103: return launch_stream<F, 2, 1, 2, 2, false, false, 3>(a, p, stream, 2);
        case 111:  // producer wave, split k; the deepest ring that leaves room for the token scales
        case 112: {
            hipError_t e = variant == 112 ? launch_stream<F, 1, 1, 0, 4, true, false, 3>(a, p, stream, 1) : hipErrorNotSupported;
            if (e == hipErrorNotSupported) e = launch_stream<F, 1, 1, 0, 3, true, false, 3>(a, p, stream, 1);
            return e != hipErrorNotSupported ? e : launch_stream<F, 1, 1, 0, 2, true, false, 3>(a, p, stream, 1);
        }
        case 116: return launch_stream<F, 1, 1, 0, 2, true, false, 3>(a, p, stream, 1);
        default: break;
        }
        if (rows > 64) return launch_stream<F, 2, 1, 2, 2, false, false, 2>(a, p, stream, 2);
        if (rows > 32) return hipErrorNotSupported;  // 33..64 tokens: the tile kernel's 64-token split-k shape
        const hipError_t e = launch_stream<F, 1, 1, 0, 3, true, false, 3>(a, p, stream, 1);
        return e != hipErrorNotSupported ? e : launch_stream<F, 1, 1, 0, 2, true, false, 3>(a, p, stream, 1);
    }
}

}  // namespace oxq
