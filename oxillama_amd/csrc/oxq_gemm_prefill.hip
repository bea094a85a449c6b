// Prefill matmul (many token rows) for the K-quants whose scaled weights are exact in f16:
//   out[m x n] (+)= A_q8[m rows of Q8_0 blocks] x W[n x k]^T,   W in Q4_K
// i.e. m fused matvecs over the same weight blocks (the reference's gemm is that loop,
// crates/oxillama-quant/src/reference/q4_k.rs:186-201, with matvec_q8_fused's arithmetic, :218-333).
//
// Why a second kernel beside the int8 tile kernel (oxq_gemm_tile.hpp): there every int32 result of the matrix
// core needs two fp32 operations (weight scale, token scale), and that vector work, not the matrix core, bounds
// the kernel.  Here the 6-bit sub-block scale rides inside the weight operand: sc * q <= 63 * 15 = 945 is exact
// in f16, the Q8_0 payload is exact in f16, and two v_mfma_f32_32x32x16_f16 with a zero addend give
// sc * I[token][row][sub-block] exactly in fp32 (< 2^24).  One fma per result applies the token's block scale;
// d and dmin are applied once per 256-weight super-block:
//   y[t][r] = sum_blk ( d[r][blk] * sum_s da[t][s] * (sc[r][s] * I[t][r][s])  -  dmin[r][blk] * sum_s mn[r][s] * P[t][s] )
// with P = da * sum(q_a) (fp32, exact).  The second sum is one more small matrix product per super-block: P is
// split exactly into three bf16 pieces (8 + 8 + 8 bits) and mn (<= 63) is exact in bf16, so two
// v_mfma_f32_32x32x16_bf16 per tile and super-block form it with fp32 accumulation.
//
// Layout of the work: a work group is 8 waves (two per SIMD, one work group per compute unit), 128 tokens x 256
// weight rows; wave w owns rows 32w..32w+31 against all 128 tokens (four 32 x 32 tiles).  The weight side is the
// MFMA's A operand, the token side its B operand, so a lane's 16 results of a tile belong to ONE token (column)
// and 16 rows: the token scale of the fma is a single register, and the per-row factors d, dmin are read once per
// super-block.
//  * weights: lane (row c, half h) fetches its row's 16 bytes of a 64-weight group straight from HBM / L2 (one
//    buffer load per group, a whole super-block ahead) and unpacks them in registers: nibble pairs are masked into
//    the mantissa of f16 1024.0 (one v_and_or per two weights) and one packed f16 fma per two weights turns
//    1024 + q (or 1024 + 16 q for the high nibbles) into sc * q exactly.  Every weight is unpacked once per work group.
//  * tokens: the preparation kernel writes the Q8_0 payload as f16 in operand order; a stage (one 64-weight group)
//    of the work group's 128 tokens is 16 KB and reaches LDS by direct-to-LDS loads into one of four buffers (one
//    per group of a super-block), requested three stages before it is read; one work-group barrier per stage; the
//    eight waves read the same fragments from LDS (conflict-free 16-byte reads).
//  * the loop is one software pipeline over the 32 (sub-block, token tile) steps of a super-block, written out
//    through a compile-time index: at step q the matrix core gets step q + 1, LDS is asked for step q + 2, the
//    fmas consume step q, and the unpacking of the operands that come next is spread over the steps; the first
//    operands of a stage are fetched during the stage before, so nothing waits at the barrier but the barrier.
// What bounds it, measured on the part with instruction mixes of this shape (two waves per SIMD, every SIMD busy):
// two such MFMAs alone take 35.8 ns per step, 16 fmas alone 22.7 ns, both together 57.5 ns -- the sum, not the
// maximum: matrix and vector work do not overlap here beyond the first eight fmas.  The int8 form's step (one int8
// MFMA 16.4 ns + 32 fmas 45.4 ns) is 61.8 ns by the same count, so this form's advantage is the unpacking and
// scale handling it saves, not a factor of two.
#include <utility>
#include "oxq_gemm_tile.hpp"

namespace oxq {

template <class F, int... Q>
__device__ __forceinline__ void static_for(std::integer_sequence<int, Q...>, F &&f) {
    (f(std::integral_constant<int, Q>{}), ...);
}

typedef _Float16 h8 __attribute__((ext_vector_type(8)));
typedef _Float16 h2v __attribute__((ext_vector_type(2)));
typedef __bf16 b8 __attribute__((ext_vector_type(8)));
typedef float v4f __attribute__((ext_vector_type(4)));

#define OXQ_LDS_PTR(p) ((__attribute__((address_space(3))) void *)(p))

// LDS is carved out of byte arrays here and written with one vector type and read with another (and filled by
// direct-to-LDS loads): every such access goes through a may_alias type, or type-based alias analysis treats a
// load as unrelated to the store that feeds it.
typedef u32x4 __attribute__((may_alias)) lds_u32x4;
typedef u32x2 __attribute__((may_alias)) lds_u32x2;
typedef uint32_t __attribute__((may_alias)) lds_u32;
typedef uint16_t __attribute__((may_alias)) lds_u16;
typedef float __attribute__((may_alias)) lds_f32;
typedef v4f __attribute__((may_alias)) lds_v4f;
__device__ __forceinline__ h8 lds_h8(const uint8_t *p) { return __builtin_bit_cast(h8, *reinterpret_cast<const lds_u32x4 *>(p)); }
__device__ __forceinline__ b8 lds_b8(const uint8_t *p) { return __builtin_bit_cast(b8, *reinterpret_cast<const lds_u32x4 *>(p)); }

constexpr uint32_t PF_TOK = 128, PF_ROWS = 256, PF_WAVES = 8;   // tokens, weight rows and waves of a work group
constexpr uint32_t PF_STAGE = 16384;              // f16 token operands of one stage: 2 sub-blocks x 128 tokens x 32 x 2 B
constexpr uint32_t PF_STAGE_DA = 512;             // + the tokens' two block scales (f16 pairs)

// Workspace planes for mpad tokens (a multiple of 128) and nsb = k/32 sub-blocks:
//   tokf  [nsb][mpad/32][half h][kk][token c][8 f16]   the Q8_0 payload as f16, k-slots in operand order
//   dag   [nsb/2][mpad][2 f16]                          block scales of the two sub-blocks of a 64-weight group
//   pbf   [nsb/8][4][mpad][8 bf16]                      per super-block: the three bf16 pieces of P for its eight
//                                                       sub-blocks, and a plane of zeros
__host__ __device__ inline size_t pf_tokf_bytes(size_t nsb, size_t mpad) { return nsb * mpad * 64; }
__host__ __device__ inline size_t pf_dag_bytes(size_t nsb, size_t mpad) { return nsb / 2 * mpad * 4; }
__host__ __device__ inline size_t pf_pbf_bytes(size_t nsb, size_t mpad) { return nsb / 8 * 4 * mpad * 16; }

// Order of the eight k-slots of one operand register set: byte positions of the lane's 8 raw weight bytes.  The
// unpack takes bytes 0 and 2 of a dword together (they sit in the two 16-bit halves), then bytes 1 and 3.
__device__ __forceinline__ constexpr int pf_slot_byte(int j) { return (j & 4) | ((j & 1) << 1) | ((j >> 1) & 1); }

// One thread per (sub-block j, token t).  Eight consecutive threads take the eight sub-blocks of one super-block of one
// token (272 contiguous bytes of its row; their eight bf16 pieces of P make one 16-byte run), the next eight the next
// token: reads in runs of a row's bytes, operand writes in runs of eight tokens per sub-block.
__global__ __launch_bounds__(256) void prefill_prep_acts(const uint8_t *__restrict__ A, uint8_t *__restrict__ tokf,
                                                        uint16_t *__restrict__ dag, uint16_t *__restrict__ pbf, uint32_t m,
                                                        uint32_t mpad, uint32_t nsb) {
    const uint32_t idx = blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= mpad * nsb) return;
    const uint32_t grp = idx >> 3, t = grp % mpad, j = (grp / mpad) * 8 + (idx & 7);
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
    const uint32_t tt = t >> 5, c = t & 31, TT = mpad >> 5;
#pragma unroll
    for (int h = 0; h < 2; h++)
#pragma unroll
        for (int kk = 0; kk < 2; kk++) {
            h8 v;
#pragma unroll
            for (int e = 0; e < 8; e++) {
                const int byte = 8 * kk + pf_slot_byte(e);
                v[e] = (_Float16)(int)(int8_t)((q[h][byte >> 2] >> (8 * (byte & 3))) & 0xFF);
            }
            *reinterpret_cast<h8 *>(tokf + (((((size_t)j * TT + tt) * 2 + h) * 2 + kk) * 32 + c) * 16) = v;
        }
    dag[((size_t)(j >> 1) * mpad + t) * 2 + (j & 1)] = (uint16_t)dbits;
    // P = da * sum(q): at most 23 significant bits; three truncated bf16 pieces hold it exactly
    const float P = h2f(dbits) * (float)s;
    const uint32_t pb = __builtin_bit_cast(uint32_t, P);
    const float p1 = __builtin_bit_cast(float, pb & 0xFFFF0000u);
    const float r1 = P - p1;  // exact
    const float p2 = __builtin_bit_cast(float, __builtin_bit_cast(uint32_t, r1) & 0xFFFF0000u);
    const float r2 = r1 - p2;  // exact, at most 8 significant bits
    const size_t pbase = (size_t)(j >> 3) * 4 * mpad;
    pbf[((pbase + 0 * (size_t)mpad + t) * 8) + (j & 7)] = (uint16_t)(pb >> 16);
    pbf[((pbase + 1 * (size_t)mpad + t) * 8) + (j & 7)] = (uint16_t)(__builtin_bit_cast(uint32_t, p2) >> 16);
    pbf[((pbase + 2 * (size_t)mpad + t) * 8) + (j & 7)] = (uint16_t)(__builtin_bit_cast(uint32_t, r2) >> 16);
    pbf[((pbase + 3 * (size_t)mpad + t) * 8) + (j & 7)] = 0;
}

// Per-wave tables of one super-block of the wave's 32 rows, in LDS:
//   sck  [group g][row][c1 lo, c2 lo, c1 hi, c2 hi]  f16 pairs: the unpack's fma constants of sub-blocks 2g (low
//        nibbles: sc, -1024 sc) and 2g+1 (high nibbles: sc/16, -64 sc)
//   mnb  [row][8 bf16]  the eight 6-bit mins
//   drow [row] d,  ndm [row] -dmin   (fp32)
constexpr uint32_t PF_TAB_SCK = 0, PF_TAB_MNB = 2048, PF_TAB_D = 2560, PF_TAB_NDM = 2688, PF_TAB_BYTES = 2816;

__device__ __forceinline__ uint32_t f16x2_of(float v) {
    const uint32_t b = f2h(v);
    return b | (b << 16);
}

template <bool DUMP>
__global__ __launch_bounds__(512) __attribute__((amdgpu_waves_per_eu(2, 2))) void gemm_prefill_q4k(
    const uint8_t *__restrict__ W, const uint8_t *__restrict__ tokf, const uint8_t *__restrict__ dag,
    const uint8_t *__restrict__ pbf, float *__restrict__ out, int32_t *__restrict__ sums, uint32_t m, uint32_t mpad,
    uint32_t n, uint32_t k, int accumulate, const float *__restrict__ bias, uint32_t m_tiles, uint32_t n_tiles) {
    // separate arrays, one per group of a super-block: the compiler tracks direct-to-LDS loads in flight per
    // variable, and a read of one stage's buffer must not wait for the loads that fill the others
    __shared__ __align__(16) uint8_t tok0[PF_STAGE + PF_STAGE_DA];
    __shared__ __align__(16) uint8_t tok1[PF_STAGE + PF_STAGE_DA];
    __shared__ __align__(16) uint8_t tok2[PF_STAGE + PF_STAGE_DA];
    __shared__ __align__(16) uint8_t tok3[PF_STAGE + PF_STAGE_DA];
    __shared__ __align__(16) uint8_t pl[8192];
    __shared__ __align__(16) uint8_t tab[PF_WAVES][2][PF_TAB_BYTES];  // per wave, two super-blocks' tables in turn

    const uint32_t nblk = k / 256, nsb = k / 32, TT = mpad >> 5;
    const uint32_t tid = threadIdx.x, lane = tid & 63;
    const uint32_t wave = (uint32_t)__builtin_amdgcn_readfirstlane((int)(tid >> 6));
    const uint32_t c = lane & 31, h = lane >> 5;

    // work groups of one set of weight rows (all token tiles) get consecutive ids on one XCD (ids are dealt
    // round-robin to the 8 XCDs), so that their weight reads meet in that XCD's L2
    const uint32_t xcd = blockIdx.x & 7, loc = blockIdx.x >> 3;
    const uint32_t n_tile = (loc / m_tiles) * 8 + xcd, m_tile = loc % m_tiles;
    if (n_tile >= n_tiles) return;
    const uint32_t m_wg = m_tile * PF_TOK, n_wg = n_tile * PF_ROWS, n_wave = n_wg + 32 * wave;
    const uint32_t tt0 = m_wg >> 5;

    const uint32_t row_bytes = nblk * 144;
    const uint32_t n_base = min(n_wg, n - 1);
    const size_t w_left = (size_t)(n - n_base) * row_bytes;
    const __amdgpu_buffer_rsrc_t rs_w = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<uint8_t *>(W + (size_t)n_base * row_bytes), 0, (int)min(w_left, (size_t)0x7FFFFFFF), BUFFER_FLAGS);
    const __amdgpu_buffer_rsrc_t rs_t = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<uint8_t *>(tokf), 0, (int)pf_tokf_bytes(nsb, mpad), BUFFER_FLAGS);
    const __amdgpu_buffer_rsrc_t rs_d = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<uint8_t *>(dag), 0, (int)pf_dag_bytes(nsb, mpad), BUFFER_FLAGS);
    const __amdgpu_buffer_rsrc_t rs_p = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<uint8_t *>(pbf), 0, (int)pf_pbf_bytes(nsb, mpad), BUFFER_FLAGS);
    // the lane's weight row as A-operand supplier (rows past n re-read the last row; their results are not stored)
    const uint32_t wrow_off = (min(n_wave + c, n - 1) - n_base) * row_bytes;

    // ---- direct-to-LDS requests -------------------------------------------------------------------------------
    // stage S = 4 * blk + g: the f16 payload of sub-blocks 2S and 2S + 1 for the work group's four token tiles
    // (2 x 8 KB, each contiguous in the workspace), 1 KB per wave and request; then the 128 tokens' scale pairs.
    // (No branch in here, nor anywhere in the loop: its body must stay one basic block, or the compiler sinks the
    // accumulate fmas of every stage down to the super-block's end and spills the matrix core's results; the waves
    // repeat the request of the scale pairs, the same bytes to the same place.)
    auto request_stage = [&](uint8_t *buf, uint32_t S) __attribute__((always_inline)) {
#pragma unroll
        for (uint32_t e = 0; e < 2; e++)
            __builtin_amdgcn_raw_ptr_buffer_load_lds(rs_t, OXQ_LDS_PTR(buf + (8 * e + wave) * 1024), 16, lane * 16,
                                                     ((2 * S + e) * TT + tt0) * 2048 + wave * 1024, 0, 0);
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rs_d, OXQ_LDS_PTR(buf + PF_STAGE + (wave & 1) * 256), 4, lane * 4,
                                                 (S * mpad + m_wg + (wave & 1) * 64) * 4, 0, 0);
    };
    // the bf16 pieces of P of one super-block: plane wave / 2 (2 KB: 128 tokens x 16 B), half wave % 2
    auto request_p = [&](uint32_t blk) __attribute__((always_inline)) {
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rs_p, OXQ_LDS_PTR(pl + wave * 1024), 16, lane * 16,
                                                 ((blk * 4 + (wave >> 1)) * mpad + m_wg + 64 * (wave & 1)) * 16, 0, 0);
    };
    // End of stage S.  The next stage reads the buffer of stage S + 2 before ITS end (the first operands of a stage
    // are fetched during the stage before), so every wave's requests for that buffer must have landed here: they
    // were issued at the start of stage S - 1, and at least five vector-memory operations of this wave follow them
    // (the weight load of that stage; three requests and a weight load of this one), which return in order.  The
    // requests of this stage stay in flight across the barrier.  The barrier also frees this stage's buffer for the
    // request that opens the next stage.
    auto stage_end = [&]() __attribute__((always_inline)) {
        __builtin_amdgcn_sched_barrier(0);
        asm volatile("s_waitcnt vmcnt(4) lgkmcnt(0)\n\ts_barrier" ::: "memory");
        __builtin_amdgcn_sched_barrier(0);
    };
    auto tokbuf = [&](int g) __attribute__((always_inline)) -> uint8_t * {
        return (g & 3) == 0 ? tok0 : (g & 3) == 1 ? tok1 : (g & 3) == 2 ? tok2 : tok3;
    };

    // ---- per-wave scale tables -----------------------------------------------------------------------------------
    // decode lane: row lane % 32, sub-blocks 4 * (lane / 32) .. + 3 (decode_scales_mins, reference/q4_k.rs:27-49)
    auto decode = [&](const u32x4 hd, uint8_t *tabw) __attribute__((always_inline)) {
        const float d = h2f(hd[0] & 0xFFFF), dmin = h2f(hd[0] >> 16);
        uint32_t mnq[2];
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const uint32_t s = 4 * h + i, sh = 8 * i;
            const uint32_t sc_lo = (hd[1] >> sh) & 63, mn_lo = (hd[2] >> sh) & 63;
            const uint32_t sc_hi = ((hd[3] >> sh) & 15) | (((hd[1] >> (sh + 6)) & 3) << 4);
            const uint32_t mn_hi = ((hd[3] >> (sh + 4)) & 15) | (((hd[2] >> (sh + 6)) & 3) << 4);
            const uint32_t sc = h ? sc_hi : sc_lo, mn = h ? mn_hi : mn_lo;
            const float fs = (float)sc;
            // sub-block s = 2g + e: e = 0 takes the low nibbles (1024 + q), e = 1 the high ones (1024 + 16 q)
            const uint32_t g = s >> 1, e = s & 1;
            u32x2 ck;
            ck[0] = f16x2_of(e ? fs * 0.0625f : fs);
            ck[1] = f16x2_of(e ? -64.0f * fs : -1024.0f * fs);
            *reinterpret_cast<lds_u32x2 *>(tabw + PF_TAB_SCK + (g * 32 + c) * 16 + e * 8) = ck;
            const uint32_t mb = __builtin_bit_cast(uint32_t, (float)mn) >> 16;  // bf16 of an integer <= 63: exact
            if (i & 1) mnq[i >> 1] |= mb << 16; else mnq[i >> 1] = mb;
        }
        *reinterpret_cast<lds_u32x2 *>(tabw + PF_TAB_MNB + c * 16 + h * 8) = u32x2{mnq[0], mnq[1]};
        // (both halves write the row's d and -dmin: the same values to the same place, and no branch)
        *reinterpret_cast<lds_f32 *>(tabw + PF_TAB_D + c * 4) = d;
        *reinterpret_cast<lds_f32 *>(tabw + PF_TAB_NDM + c * 4) = -dmin;
    };

    v16f y[4], accblk[4];
    for (int a = 0; a < 4; a++)
        for (int i = 0; i < 16; i++) y[a][i] = 0.0f, accblk[a][i] = 0.0f;
    v16f zero16;
    for (int i = 0; i < 16; i++) zero16[i] = 0.0f;
    // masks in scalar registers and the f16 1024.0 pair in a vector register, hidden from constant folding: (w & mask)
    // | magic is then ONE v_and_or_b32 (the instruction takes one scalar operand and no second literal)
    uint32_t mask_lo = 0x000F000Fu, mask_hi = 0x00F000F0u, magic = 0x64006400u;
    asm volatile("" : "+s"(mask_lo), "+s"(mask_hi), "+v"(magic));

    // weight bytes: slot g holds the lane's 16 bytes of group g of the current super-block; it is refilled with the
    // next super-block's once both of its sub-blocks are unpacked
    u32x4 wq[4];
    auto fetch_w = [&](uint32_t blk, uint32_t g) __attribute__((always_inline)) {
        return buf16(rs_w, wrow_off + 16 * h, min(blk, nblk - 1) * 144 + 16 + 32 * g);
    };
    // A operands of one sub-block from the lane's 16 raw bytes: low nibbles (1024 + q) * sc - 1024 sc, or high
    // nibbles in place (1024 + 16 q) * sc/16 - 64 sc: sc * q exactly.  kk: which 8 bytes.
    auto unpack = [&](const u32x4 raw, int kk, uint32_t mask, uint32_t k1, uint32_t k2) __attribute__((always_inline)) {
        const h2v c1 = __builtin_bit_cast(h2v, k1), c2 = __builtin_bit_cast(h2v, k2);
        uint32_t o[4];
#pragma unroll
        for (int d = 0; d < 2; d++) {
            const uint32_t w = raw[2 * kk + d], w8 = w >> 8;
            const h2v t0 = __builtin_bit_cast(h2v, (w & mask) | magic);   // bytes 0 and 2 of the dword
            const h2v t1 = __builtin_bit_cast(h2v, (w8 & mask) | magic);  // bytes 1 and 3
            o[2 * d] = __builtin_bit_cast(uint32_t, __builtin_elementwise_fma(t0, c1, c2));
            o[2 * d + 1] = __builtin_bit_cast(uint32_t, __builtin_elementwise_fma(t1, c1, c2));
        }
        return __builtin_bit_cast(h8, u32x4{o[0], o[1], o[2], o[3]});
    };
    auto tok_frag = [&](const uint8_t *buf, int ts, int kk) __attribute__((always_inline)) {
        return lds_h8(buf + (((ts * 2 + h) * 2 + kk) * 32 + c) * 16);
    };
    // block scale (f16 bits) of the lane's token of tile mt for sub-block e of the stage in `buf`
    auto tok_scale = [&](const uint8_t *buf, int e, int mt) __attribute__((always_inline)) {
        return (uint32_t)*reinterpret_cast<const lds_u16 *>(buf + PF_STAGE + (mt * 32 + c) * 4 + 2 * e);
    };

    // ---- fill the pipeline ------------------------------------------------------------------------------------------
#pragma unroll
    for (int g = 0; g < 4; g++) wq[g] = fetch_w(0, g);
    decode(buf16(rs_w, wrow_off, 0), tab[wave][0]);
    request_stage(tok0, 0);
    request_stage(tok1, min(1u, 4 * nblk - 1));
    request_stage(tok2, min(2u, 4 * nblk - 1));
    __syncthreads();
    // state carried from step to step (q = 8 g + ts: sub-block 2g + ts / 4 against token tile ts % 4):
    //   wf[e]   A operands of sub-block e of the current group (wf[0] of the NEXT group from step 4 on)
    //   ck      fma constants of the sub-block whose operands are unpacked next
    //   tf[i]   token fragments of step q + 1 (i = (q + 1) % 2) and, once requested, q + 2
    //   dah[i]  block scale of the lane's token for step q (i = q % 2) and q + 1
    //   T[i]    matrix-core results of step q (i = q % 2) and q + 1
    h8 wf[2][2], tf[2][2];
    v16f T[2];
    uint32_t dah[2];
    u32x2 ck;  // fma constants (c1, c2) of the sub-block unpacked next
    ck = *reinterpret_cast<const lds_u32x2 *>(tab[wave][0] + PF_TAB_SCK + c * 16);
    wf[0][0] = unpack(wq[0], 0, mask_lo, ck[0] + 0u, ck[1] + 0u);
    wf[0][1] = unpack(wq[0], 1, mask_lo, ck[0] + 0u, ck[1] + 0u);
    ck = *reinterpret_cast<const lds_u32x2 *>(tab[wave][0] + PF_TAB_SCK + c * 16 + 8);
    dah[0] = tok_scale(tok0, 0, 0);
    tf[0][0] = tok_frag(tok0, 0, 0);
    tf[0][1] = tok_frag(tok0, 0, 1);
    tf[1][0] = tok_frag(tok0, 1, 0);
    tf[1][1] = tok_frag(tok0, 1, 1);
    T[0] = __builtin_amdgcn_mfma_f32_32x32x16_f16(wf[0][0], tf[0][0], zero16, 0, 0, 0);
    T[0] = __builtin_amdgcn_mfma_f32_32x32x16_f16(wf[0][1], tf[0][1], T[0], 0, 0, 0);

    for (uint32_t blk = 0; blk < nblk; blk++) {
        const uint32_t S0 = 4 * blk, Slast = 4 * nblk - 1;
        uint8_t *const tab_cur = tab[wave][blk & 1], *const tab_next = tab[wave][(blk + 1) & 1];
        u32x4 hd_next;
        // (32 steps written out through a compile-time index: `#pragma unroll` gives up on a body this size, and every
        // register array below is indexed by the step)
        static_for(std::make_integer_sequence<int, 32>{}, [&](auto qc) __attribute__((always_inline)) {
            constexpr int q = decltype(qc)::value;
            constexpr int g = q >> 3, ts = q & 7, e = ts >> 2, mt = ts & 3;
            if constexpr (ts == 0) {
                // the buffer of the stage before is free since the barrier that ended it: it takes the stage three ahead
                request_stage(tokbuf(g + 3), min(S0 + g + 3, Slast));
                if constexpr (g == 0) {
                    request_p(blk);  // read at this super-block's end; the previous one's end read pl before its barrier
                    hd_next = buf16(rs_w, wrow_off, min(blk + 1, nblk - 1) * 144);
                }
            }
            // matrix core: step q + 1 (the first step of the next group uses the operands unpacked during this one)
            {
                const int q1 = q + 1, e1 = (q1 & 7) >> 2;
                T[q1 & 1] = __builtin_amdgcn_mfma_f32_32x32x16_f16(wf[e1][0], tf[q1 & 1][0], zero16, 0, 0, 0);
                T[q1 & 1] = __builtin_amdgcn_mfma_f32_32x32x16_f16(wf[e1][1], tf[q1 & 1][1], T[q1 & 1], 0, 0, 0);
            }
            // token fragments of step q + 2, into the slot that step q's matrix instructions have read
            {
                const int q2 = q + 2;
                const uint8_t *const b2 = tokbuf(q2 >> 3);
                tf[q & 1][0] = tok_frag(b2, q2 & 7, 0);
                tf[q & 1][1] = tok_frag(b2, q2 & 7, 1);
            }
            {
                constexpr int q1 = q + 1;
                dah[q1 & 1] = tok_scale(tokbuf(q1 >> 3), (q1 & 7) >> 2, q1 & 3);
            }
            // this step's results: accblk += da * (sc * I)
            const float da = h2f(dah[q & 1]);
            const v16f t = T[q & 1];
#pragma unroll
            for (int i = 0; i < 16; i++) accblk[mt][i] = q < 4 ? t[i] * da : fmaf(t[i], da, accblk[mt][i]);  // (a tile's first step of the super-block starts its sum)
            if constexpr (DUMP) {
                const uint32_t tok = m_wg + mt * 32 + c;
#pragma unroll
                for (int i = 0; i < 16; i++) {
                    const uint32_t row = n_wave + 8 * (i >> 2) + 4 * h + (i & 3);
                    if (tok < m && row < n) sums[((size_t)tok * n + row) * nsb + blk * 8 + 2 * g + e] = (int)t[i];
                }
            }
            // operand preparation, spread over the steps: the high nibbles of this group (needed from step 4 on),
            // then the low nibbles of the next group (wf[0] is free once step 3's matrix instructions are issued)
            if constexpr (ts == 0) wf[1][0] = unpack(wq[g], 0, mask_hi, ck[0] + 0u, ck[1] + 0u);
            if constexpr (ts == 1) wf[1][1] = unpack(wq[g], 1, mask_hi, ck[0] + 0u, ck[1] + 0u);
            if constexpr (ts == 2) {
                wq[g] = fetch_w(blk + 1, g);
                if constexpr (g == 1) decode(hd_next, tab_next);
            }
            if constexpr (ts == 3 || ts == 6)  // the next group's constants: low nibbles' pair, later the high nibbles'
                ck = *reinterpret_cast<const lds_u32x2 *>((g == 3 ? tab_next : tab_cur) + PF_TAB_SCK +
                                                          (((g + 1) & 3) * 32 + c) * 16 + (ts == 6 ? 8 : 0));
            if constexpr (ts == 4) wf[0][0] = unpack(wq[(g + 1) & 3], 0, mask_lo, ck[0] + 0u, ck[1] + 0u);
            if constexpr (ts == 5) wf[0][1] = unpack(wq[(g + 1) & 3], 1, mask_lo, ck[0] + 0u, ck[1] + 0u);
            if constexpr (q >= 28) {
                // ---- the super-block's factors for token tile mt, whose last step this was:
                //      y += d * accblk - dmin * (mn . P) -------------------------------------------------------------
                const b8 mn8 = lds_b8(tab_cur + PF_TAB_MNB + c * 16);
                const b8 pa = lds_b8(pl + ((h * 4 + mt) * 32 + c) * 16);
                const b8 pb = lds_b8(pl + (((2 + h) * 4 + mt) * 32 + c) * 16);
                v16f U = __builtin_amdgcn_mfma_f32_32x32x16_bf16(mn8, pa, zero16, 0, 0, 0);
                U = __builtin_amdgcn_mfma_f32_32x32x16_bf16(mn8, pb, U, 0, 0, 0);
#pragma unroll
                for (int a = 0; a < 4; a++) {
                    const v4f dv = *reinterpret_cast<const lds_v4f *>(tab_cur + PF_TAB_D + (8 * a + 4 * h) * 4);
                    const v4f nv = *reinterpret_cast<const lds_v4f *>(tab_cur + PF_TAB_NDM + (8 * a + 4 * h) * 4);
#pragma unroll
                    for (int b = 0; b < 4; b++) {
                        y[mt][4 * a + b] = fmaf(accblk[mt][4 * a + b], dv[b], y[mt][4 * a + b]);
                        y[mt][4 * a + b] = fmaf(U[4 * a + b], nv[b], y[mt][4 * a + b]);
                    }
                }
            }
            __builtin_amdgcn_sched_barrier(0);
            if constexpr (ts == 7) stage_end();
        });
    }
    __syncthreads();  // every request has landed before the work group's LDS is given back

    // ---- store: lane (token c, half h) holds rows 8a + 4h + 0..3 of its wave's 32, for four token tiles ----------
    const bool vec4 = (n & 3) == 0 && (reinterpret_cast<uintptr_t>(out) & 15) == 0 &&
                      (!bias || (reinterpret_cast<uintptr_t>(bias) & 15) == 0);
#pragma unroll
    for (int mt = 0; mt < 4; mt++) {
        const uint32_t tok = m_wg + mt * 32 + c;
        if (tok >= m) continue;
#pragma unroll
        for (int a = 0; a < 4; a++) {
            const uint32_t row = n_wave + 8 * a + 4 * h;
            if (row >= n) continue;
            float *o = out + (size_t)tok * n + row;
            if (vec4) {
                v4f v = {y[mt][4 * a], y[mt][4 * a + 1], y[mt][4 * a + 2], y[mt][4 * a + 3]};
                if (accumulate) {
                    const v4f old = *reinterpret_cast<const v4f *>(o);
                    v = old + v;
                } else if (bias) {
                    v = v + *reinterpret_cast<const v4f *>(bias + row);
                }
                *reinterpret_cast<v4f *>(o) = v;
            } else {
#pragma unroll
                for (int b = 0; b < 4; b++)
                    if (row + b < n)
                        o[b] = accumulate ? o[b] + y[mt][4 * a + b] : bias ? y[mt][4 * a + b] + bias[row + b] : y[mt][4 * a + b];
            }
        }
    }
}

size_t gemm_prefill_workspace_bytes(uint32_t m, uint32_t k) {
    const size_t mpad = ((size_t)m + PF_TOK - 1) / PF_TOK * PF_TOK, nsb = k / 32;
    return pf_tokf_bytes(nsb, mpad) + pf_dag_bytes(nsb, mpad) + pf_pbf_bytes(nsb, mpad);
}

bool gemm_prefill_supported(uint32_t type, uint32_t m, uint32_t n, uint32_t k) {
    if (type != OXQ_TYPE_Q4_K || k == 0 || k % 256 != 0 || m == 0 || n == 0) return false;
    const size_t mpad = ((size_t)m + PF_TOK - 1) / PF_TOK * PF_TOK, nsb = k / 32;
    // buffer descriptors address 2^31 bytes; scalar offsets are 32-bit
    return pf_tokf_bytes(nsb, mpad) < 0x7FFFFFFFull && (size_t)(k / 256) * 144 * PF_ROWS < 0x7FFFFFFFull;
}

hipError_t launch_gemm_prefill(uint32_t type, const GemmArgs &a, hipStream_t stream) {
    if (!gemm_prefill_supported(type, a.m, a.n, a.k) || a.offsets || !a.workspace) return hipErrorNotSupported;
    const uint32_t mpad = (a.m + PF_TOK - 1) / PF_TOK * PF_TOK, nsb = a.k / 32;
    uint8_t *tokf = a.workspace;
    uint8_t *dag = tokf + pf_tokf_bytes(nsb, mpad);
    uint8_t *pbf = dag + pf_dag_bytes(nsb, mpad);
    hipLaunchKernelGGL(prefill_prep_acts, dim3((mpad * nsb + 255) / 256), dim3(256), 0, stream, a.A, tokf,
                       reinterpret_cast<uint16_t *>(dag), reinterpret_cast<uint16_t *>(pbf), a.m, mpad, nsb);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return e;
    const uint32_t m_tiles = mpad / PF_TOK, n_tiles = (a.n + PF_ROWS - 1) / PF_ROWS;
    const dim3 grid(8 * ((n_tiles + 7) / 8) * m_tiles);
    note_launch("gemm_prefill_q4k", type, a.sums ? 1 : 0, 0, 0, 0, grid.x, 1, 512);
    if (a.sums)
        hipLaunchKernelGGL(gemm_prefill_q4k<true>, grid, dim3(512), 0, stream, a.W, tokf, dag, pbf, a.out, a.sums, a.m,
                           mpad, a.n, a.k, a.accumulate, a.bias, m_tiles, n_tiles);
    else
        hipLaunchKernelGGL(gemm_prefill_q4k<false>, grid, dim3(512), 0, stream, a.W, tokf, dag, pbf, a.out, a.sums, a.m,
                           mpad, a.n, a.k, a.accumulate, a.bias, m_tiles, n_tiles);
    return hipGetLastError();
}

}  // namespace oxq
