// The batched form of the fused matvec (prefill, decode batch, mixture-of-experts group): host
// side, and the tile kernel instantiated for Q4_0, Q8_0, Q4_K, Q6_K, IQ4_XS.  Kernel and launch
// templates: oxq_gemm_tile.hpp; further formats: oxq_gemm_more.hip.
#include "oxq_gemm_skinny.hpp"

namespace oxq {

// Without the tile kernel (very few rows, or a shape it does not take): GEMV launches, two to
// four activation rows per pass over the weights where the row length allows.
static hipError_t gemm_by_rows(uint32_t type, const GemmArgs &a, hipStream_t stream) {
    // Q8_0 blocks per activation row: whole weight blocks' worth, also where a row ends inside one
    const size_t bs = oxq_block_size(type);
    const size_t act_row_bytes = ((size_t)a.k + bs - 1) / bs * (bs / 32) * 34;
    const uint32_t vecs = gemv_vecs_max(type, a.k);
    uint32_t r = 0;
    while (r < a.m) {
        const uint32_t left = a.m - r;
        if (vecs >= 2 && left >= 2) {  // 2..4 activation rows share one pass over the weights
            GemvVecsArgs v;
            v.W = a.W;
            v.A = a.A + r * act_row_bytes;
            v.a_stride = act_row_bytes;
            v.out = a.out + (size_t)r * a.n;
            v.out_stride = a.n;
            v.n_vecs = left < vecs ? left : vecs;
            v.n_rows = a.n;
            v.n_cols = a.k;
            v.accumulate = a.accumulate;
            v.bias = a.bias;
            hipError_t e = launch_gemv_vecs(type, v, stream);
            if (e != hipSuccess) return e;
            r += v.n_vecs;
            continue;
        }
        GemvArgs g;
        g.W = a.W;
        g.A = a.A + r * act_row_bytes;
        g.out = a.out + (size_t)r * a.n;
        g.sums = nullptr;
        g.n_rows = a.n;
        g.n_cols = a.k;
        g.accumulate = a.accumulate;
        g.bias = a.bias;
        g.waves_per_cu = 0;
        g.rows_per_batch = 0;
        g.waves_per_row = 0;
        hipError_t e = launch_gemv_q8(type, g, stream);
        if (e != hipSuccess) return e;
        r++;
    }
    return hipSuccess;
}

std::atomic<int> g_gemm_variant{0};  // tuning: 0 = default

static size_t gemm_planes_bytes(uint32_t m, uint32_t k) {
    // token rows are padded so that a 128-token tile starting at any row stays inside
    const size_t mpad = ((size_t)m + 127) / 128 * 128 + 128, nsb = tile_padded_sub_blocks(k);
    return nsb * mpad * (32 + 4 + 2 + 8);  // activation bytes, P, f16 scales, the two half-block planes of P
}
// The formats the few-token kernel has a policy for.
static bool gemm_few_token_format(uint32_t type) {
    return type == OXQ_TYPE_Q4_K || type == OXQ_TYPE_IQ4_XS || type == OXQ_TYPE_Q6_K || type == OXQ_TYPE_Q8_0 ||
           type == OXQ_TYPE_Q4_0 || type == OXQ_TYPE_Q5_K || type == OXQ_TYPE_Q3_K || type == OXQ_TYPE_Q4_1 ||
           type == OXQ_TYPE_IQ4_NL || type == OXQ_TYPE_Q5_0 || type == OXQ_TYPE_Q5_1 ||
           type == OXQ_TYPE_Q2_K;
}
// Bytes of the few-token kernel's per-split sums for this call, 0 if it would not split k.
static size_t gemm_partial_bytes(uint32_t type, uint32_t m, uint32_t n, uint32_t k) {
    if (!gemm_few_token_format(type) || m > 32 || (m > 16 && (n >= 8192 || (uint64_t)n * k < (1ull << 25))) || n == 0) return 0;
    const uint32_t splits = skinny_splits(n, k);
    return splits > 1 ? (size_t)splits * m * n * sizeof(float) : 0;
}
// The same for the grouped form, which splits k in two where an expert's matrix has few row groups: a function of
// (type, rows, n, k) only, as the caller sizes the workspace without the number of experts.
static size_t gemm_grouped_partial_bytes(uint32_t type, uint32_t m, uint32_t n, uint32_t k) {
    if (!gemm_few_token_format(type) || k % 1024 != 0 || n == 0 ||
        n > SKINNY_GROUPED_SPLIT_MAX_N)
        return 0;
    const size_t bytes = (size_t)2 * m * n * sizeof(float);
    return bytes <= ((size_t)64 << 20) ? bytes : 0;
}
size_t gemm_grouped_workspace_bytes(uint32_t m, uint32_t k, uint32_t n, uint32_t type) {
    const size_t planes = (gemm_planes_bytes(m, k) + 255) & ~(size_t)255;
    return planes + gemm_grouped_partial_bytes(type, m, n, k);
}
size_t gemm_workspace_bytes(uint32_t m, uint32_t k, uint32_t n, uint32_t type) {
    const size_t planes = (gemm_planes_bytes(m, k) + 255) & ~(size_t)255;
    const size_t tiles = planes + gemm_partial_bytes(type, m, n, k);
    // the prefill kernel lays its own planes (f16 token operands) over the head of the same workspace; the size is
    // a function of the shape, whichever kernel a call then takes
    const size_t prefill = gemm_prefill_supported(type, m, n ? n : 1, k) ? gemm_prefill_workspace_bytes(m, k) : 0;
    return tiles > prefill ? tiles : prefill;
}

// A plain matmul takes the prefill kernel where its work groups (128 tokens x 256 rows, one per compute unit, each
// about as long whatever the others do) fill their rounds of the chip: measured at k = 4096 against the tile
// kernel, 224 / 448 / 672 work groups on 256 compute units 110 / 202 / 298 us against 126 / 228 / 332, but 280 work
// groups 194 against 172, 168 a tie, 128 and fewer far behind (the tile kernel's smaller tiles spread better).
// And its token tiles must be mostly full: a work group costs the same with 32 of its 128 token rows in use (128256 x
// 4096: 32 / 64 / 96 / 128 tokens 208 / 220 / 234 / 245 us against 115 / 185 / 275 / 285 on the tile kernel).
static bool gemm_prefill_pays(uint32_t m, uint32_t n) {
    const uint64_t token_tiles = (m + 127) / 128;
    const uint64_t wgs = token_tiles * ((n + 255) / 256), cus = device_cus();
    const uint64_t rounds = (wgs + cus - 1) / cus;
    // (three quarters of a round still pays -- 192 work groups: 4096 x 14336 at 1536 tokens 345 us against 425, 8192 x
    // 8192 at 768 tokens 205 against 255, 6144 x 4096 at 1024 tokens 111 against 122; 560 of 768: 565 against 606 --
    // two thirds does not: 336 of 512, 14336 x 4096 at 768 tokens, 204 against 180)
    return 100 * wgs >= 72 * rounds * cus && 100 * (uint64_t)m >= 70 * 128 * token_tiles;
}

std::atomic<uint32_t> g_gemm_tile_min_rows{0};  // tuning: 0 = default

// The tile kernel can take this format and shape at all.
bool gemm_tiles_supported(uint32_t type, uint32_t m, uint32_t k) {
    // LDS holds the f16 token scales of a work group's tokens for the whole k (k/32 * 2 bytes per token) beside up
    // to 24 KB of decoded weight scales: 128-token tiles up to k = 16384, 64-token tiles up to 32768, 32-token tiles
    // up to 65536 (launch_tiles picks among them); up to k = 8192 two work groups of 128 tokens share a CU
    const bool known = type == OXQ_TYPE_Q4_K || type == OXQ_TYPE_IQ4_XS || type == OXQ_TYPE_Q6_K ||
                       type == OXQ_TYPE_Q8_0 || type == OXQ_TYPE_Q4_0 || type == OXQ_TYPE_Q5_K || type == OXQ_TYPE_Q4_1 ||
                       type == OXQ_TYPE_IQ4_NL || type == OXQ_TYPE_Q8_1 || type == OXQ_TYPE_Q5_0 || type == OXQ_TYPE_Q5_1 ||
                       type == OXQ_TYPE_Q3_K || type == OXQ_TYPE_Q2_K;
    // the 32-weight formats are walked eight blocks at a time; their rows may end inside the last eight (the
    // kernel then reads that step through the window of the row's last eight blocks), the others' may not
    const bool blocks32 = type == OXQ_TYPE_Q8_0 || type == OXQ_TYPE_Q4_0 || type == OXQ_TYPE_Q4_1 ||
                          type == OXQ_TYPE_IQ4_NL || type == OXQ_TYPE_Q8_1 || type == OXQ_TYPE_Q5_0 || type == OXQ_TYPE_Q5_1;
    const bool whole = k % 256 == 0 || (blocks32 && k % 32 == 0 && k >= 256);
    return known && whole && m >= 1 && (size_t)tile_padded_sub_blocks(k) * 64 <= 128 * 1024 &&
           gemm_planes_bytes(m, k) < 0x7FFFFFFFull;
}

// ... and is the faster way for m activation rows.  Below the threshold GEMV launches that take up
// to four rows per pass over the weights win (measured: 14336 x 4096 Q4_K, 4 rows 15 us, 8 rows 28 us
// against 22 us for the tile kernel; 4096-row matrices give the tile kernel fewer work groups:
// 4096 x 14336 Q6_K, 8 rows 41 us against 55 us, 12 rows 61 us against 55 us).
bool gemm_uses_tiles(uint32_t type, uint32_t m, uint32_t n, uint32_t k) {
    const uint32_t knob = g_gemm_tile_min_rows.load(std::memory_order_relaxed);
    // (GEMV launches of four rows per pass against the tile kernel, us: 4096 x 4096 Q4_K 6 / 8 rows 13.8 / 16.6 against
    // 12.5, Q8_0 17.5 / 23.0 against 16.9, Q6_K 20.3 / 25.0 against 17.1; 2048 x 4096 9.3 / 10.9 against 12.3)
    // 14336 x 4096, 5 rows (two GEMV passes): Q5_K 23.1 against 22.0, Q5_0 32.5 against 28.6, Q2_K 25.3 against 24.0
    const uint32_t min_rows = knob ? knob : n >= 8192 ? 5 : (uint64_t)n * k >= (1ull << 24) ? 6 : 9;
    return gemm_tiles_supported(type, m, k) && m >= min_rows;
}

// Fewer rows than that, on a shape the few-token kernel serves with k split over work groups: it still beats the
// GEMV launches, whose time grows with every four rows (measured, us, GEMV launches against the few-token kernel:
// Q4_K 14336 x 4096 4 rows 14.3 / 16.8, 5 rows 20.6 / 16.5; 4096 x 14336 5 rows 20.5 / 19.4, 8 rows 26.7 / 19.6;
// IQ4_XS 14336 x 4096 2 rows 14.1 / 16.2, 3 rows 23.2 / 16.1, 5 rows 33.2 / 16.2; 4096 x 14336 3 rows 23.3 / 19.5).
// Only where the caller has a workspace with room for the per-split sums, and with the knobs at their defaults.
bool gemm_few_rows_pay(uint32_t type, uint32_t m, uint32_t n, uint32_t k) {
    if (g_gemm_tile_min_rows.load(std::memory_order_relaxed) != 0 || g_gemm_variant.load(std::memory_order_relaxed) != 0)
        return false;
    // from 5 rows (a second GEMV pass); from 3 where a GEMV launch takes two vectors at most (rows of two or of five
    // to eight 64-lane steps: IQ4_XS and the 32-weight formats at 4096 columns, everything at 8192 and beyond --
    // Q4_K 28672 x 8192 3 / 4 rows 52.6 / 56.7 against 38.4 / 38.8, Q8_0 14336 x 4096 24.1 / 25.6 against 21.6 / 22.0)
    return gemm_tiles_supported(type, m, k) && gemm_partial_bytes(type, m, n, k) != 0 &&
           m >= (gemv_vecs_max(type, k) <= 2 ? 3u : 5u);
}

// Expert groups with at most this many token rows in all: one GEMV launch, a matvec per row against its expert's
// matrix (each row streams a whole matrix, so this pays only while rows are fewer than about the experts they hit).
// Measured on MI355X (IQ4_XS, 8 experts of Mixtral's shapes, us per matmul, GEMV launch / few-token kernel / tile
// kernel): see the table in the few-token kernel's notes.
static hipError_t gemm_grouped_by_gemv(uint32_t type, const GemmArgs &a, hipStream_t stream) {
    GemvArgs g;
    g.W = a.W;
    g.A = a.A;
    g.out = a.out;
    g.sums = nullptr;
    g.n_rows = a.n;
    g.n_cols = a.k;
    g.accumulate = a.accumulate;
    g.bias = nullptr;
    g.waves_per_cu = 0;
    g.rows_per_batch = 0;
    g.waves_per_row = 0;
    g.group_offsets = a.offsets;
    g.n_groups = a.n_experts;
    g.n_pairs = a.m;
    g.w_stride = a.w_stride;
    g.a_stride = (size_t)(a.k / 32) * 34;
    return launch_gemv_q8(type, g, stream);
}

hipError_t launch_gemm_q8(uint32_t type, const GemmArgs &a, hipStream_t stream) {
    if (a.offsets && !a.sums && !a.bias && a.m <= grouped_gemv_max_rows(a.n_experts) && a.n_experts <= 4096 &&
        g_gemm_variant.load(std::memory_order_relaxed) == 0) {
        const hipError_t e = gemm_grouped_by_gemv(type, a, stream);
        if (e != hipErrorNotSupported) return e;
    }
    const bool tiles = a.workspace != nullptr && gemm_tiles_supported(type, a.m, a.k) && (a.offsets || !a.by_rows);
    if (!tiles) {
        if (a.offsets) return hipErrorInvalidValue;  // grouped form exists for the tile kernel only
        return gemm_by_rows(type, a, stream);
    }
    const int variant = g_gemm_variant.load(std::memory_order_relaxed);
    // many token rows of a format whose scaled weights are exact in f16: the prefill kernel (oxq_gemm_prefill.hip).
    // The debug dump of the integer sums stays on the tile kernel; the dump of the scaled sums is this kernel's.
    if (!a.offsets && (variant == 0 || variant == 300) && (!a.sums || a.scaled_sums) &&
        gemm_prefill_supported(type, a.m, a.n, a.k) && a.workspace_bytes >= gemm_prefill_workspace_bytes(a.m, a.k)) {
        if (a.scaled_sums || variant == 300 || gemm_prefill_pays(a.m, a.n)) {
            const hipError_t e = launch_gemm_prefill(type, a, stream);
            if (e != hipErrorNotSupported) return e;
        }
    }
    if (a.scaled_sums) return hipErrorNotSupported;
    const uint32_t mpad = (a.m + 127) / 128 * 128 + 128, nsb = tile_padded_sub_blocks(a.k), nsb_row = a.k / 32;
    uint8_t *q8t = a.workspace;
    float *P = reinterpret_cast<float *>(q8t + (size_t)nsb * mpad * 32);
    uint16_t *da16 = reinterpret_cast<uint16_t *>(q8t + (size_t)nsb * mpad * 36);
    const dim3 pgrid((mpad * nsb + 255) / 256);
    auto act_perm = [](uint32_t t) {
        return t == OXQ_TYPE_Q6_K ? TileQ6K::ACT_PERM
               : (t == OXQ_TYPE_IQ4_XS || t == OXQ_TYPE_Q4_0) ? TileIQ4XS::ACT_PERM
               : (t == OXQ_TYPE_Q4_K || t == OXQ_TYPE_Q8_0) ? 0 : tile_act_perm_more(t);
    };
    const int perm = act_perm(type);
    TilePlan plan = {q8t, P, da16, mpad};
    if (!a.offsets && gemm_partial_bytes(type, a.m, a.n, a.k) &&
        a.workspace_bytes >= gemm_workspace_bytes(a.m, a.k, a.n, type))
        plan.partial = reinterpret_cast<float *>(a.workspace + ((gemm_planes_bytes(a.m, a.k) + 255) & ~(size_t)255));
    if (a.offsets && gemm_grouped_partial_bytes(type, a.m, a.n, a.k) &&
        a.workspace_bytes >= gemm_grouped_workspace_bytes(a.m, a.k, a.n, type))
        plan.partial = reinterpret_cast<float *>(a.workspace + ((gemm_planes_bytes(a.m, a.k) + 255) & ~(size_t)255));
    // The few-token kernel (oxq_gemm_skinny.hpp), where it pays: it reads the caller's Q8_0 rows itself, no re-layout.
    const uint32_t rows = a.offsets ? (a.shape_rows ? a.shape_rows : a.max_rows) : a.m;
    auto skinny_of = [&](uint32_t t) {
        return t == OXQ_TYPE_Q4_K     ? skinny_shape<TileQ4K>(a, plan.partial != nullptr, rows, variant)
               : t == OXQ_TYPE_IQ4_XS ? skinny_shape<TileIQ4XS>(a, plan.partial != nullptr, rows, variant)
               : t == OXQ_TYPE_Q6_K   ? skinny_shape<TileQ6K>(a, plan.partial != nullptr, rows, variant)
               : t == OXQ_TYPE_Q8_0   ? skinny_shape<TileQ8_0>(a, plan.partial != nullptr, rows, variant)
               : t == OXQ_TYPE_Q4_0   ? skinny_shape<TileQ4_0>(a, plan.partial != nullptr, rows, variant)
                                      : skinny_shape_more(t, a, plan.partial != nullptr, rows, variant);
    };
    if (const int shape = skinny_of(type)) {
        const hipError_t e = type == OXQ_TYPE_Q4_K     ? launch_skinny<TileQ4K>(a, plan, stream, shape)
                             : type == OXQ_TYPE_IQ4_XS ? launch_skinny<TileIQ4XS>(a, plan, stream, shape)
                             : type == OXQ_TYPE_Q6_K   ? launch_skinny<TileQ6K>(a, plan, stream, shape)
                             : type == OXQ_TYPE_Q8_0   ? launch_skinny<TileQ8_0>(a, plan, stream, shape)
                             : type == OXQ_TYPE_Q4_0   ? launch_skinny<TileQ4_0>(a, plan, stream, shape)
                                                       : launch_skinny_more(type, a, plan, stream, shape);
        if (e != hipErrorNotSupported) return e;
    }
    // an earlier call of the same sequence left these activations in the workspace in the byte order this format
    // needs (with the half-block planes if it needs them): go straight to the tile kernel
    const bool need_p16 = tile_needs_p16_more(type);
    const bool prepared = a.prep_state && a.prep_state->valid && a.prep_state->perm == perm &&
                          (!need_p16 || a.prep_state->p16);
    if (!prepared) {
        // formats with a 16-weight zero-point term also need P per half block
        float *p16 = need_p16
                         ? reinterpret_cast<float *>(reinterpret_cast<uint8_t *>(P) + tile_p16_offset(nsb, mpad))
                         : nullptr;
        if (perm == 2)
            hipLaunchKernelGGL(gemm_prep_acts<2>, pgrid, dim3(256), 0, stream, a.A, q8t, P, da16, a.m, mpad, nsb, p16, nsb_row);
        else if (perm == 1)
            hipLaunchKernelGGL(gemm_prep_acts<1>, pgrid, dim3(256), 0, stream, a.A, q8t, P, da16, a.m, mpad, nsb, p16, nsb_row);
        else
            hipLaunchKernelGGL(gemm_prep_acts<0>, pgrid, dim3(256), 0, stream, a.A, q8t, P, da16, a.m, mpad, nsb, p16, nsb_row);
        hipError_t e = hipGetLastError();
        if (e != hipSuccess) return e;
        if (a.prep_state) *a.prep_state = GemmArgs::Prepared{true, perm, need_p16};
    }
    switch (type) {
    case OXQ_TYPE_Q4_K: return launch_tiles<TileQ4K>(a, plan, stream);
    case OXQ_TYPE_IQ4_XS: return launch_tiles<TileIQ4XS>(a, plan, stream);
    case OXQ_TYPE_Q6_K: return launch_tiles<TileQ6K>(a, plan, stream);
    case OXQ_TYPE_Q8_0: return launch_tiles<TileQ8_0>(a, plan, stream);
    case OXQ_TYPE_Q4_0: return launch_tiles<TileQ4_0>(a, plan, stream);
    default: return launch_tiles_more(type, a, plan, stream);
    }
}

}  // namespace oxq
