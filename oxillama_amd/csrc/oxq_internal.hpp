// Host-side declarations shared by the kernel translation units and the C ABI.
#pragma once
#include <hip/hip_runtime.h>
#include <atomic>
#include <stddef.h>
#include <stdint.h>

#include "../../include/oxq.h"
#include "../../include/oxq_tuning.h"

// A weight matrix resident in HBM (oxq_weights_t): raw GGUF blocks, row-major.
struct oxq_weights {
    uint32_t type;
    size_t n_rows, n_cols, nbytes;
    uint8_t *dev;
};

namespace oxq {

// Record the calling thread's error detail (what oxq_last_error reports) and return `status`.
int set_error(int status, size_t a, size_t b, const char *msg);
// oxq_init(0) unless a device is already initialised.
int ensure_device();
// GGUF loader: pinned staging buffers, released at shutdown.
void gguf_release_staging();

struct GemvArgs {
    const uint8_t *W;     // raw GGUF blocks, row-major, device memory
    const uint8_t *A;     // Q8_0 activation blocks, device memory
    const float *X = nullptr;  // instead of A: fp32 activations, quantized to Q8_0 inside the kernel
    float *out;           // n_rows floats, device memory
    int32_t *sums;        // optional: per-row integer group sums (debug), else null
    uint32_t n_rows;
    uint32_t n_cols;      // multiple of the format's block size
    int accumulate;       // 1: out[r] += y (matvec_q8_fused), 0: out[r] = y (gemv)
    const float *bias = nullptr;  // with accumulate == 0: out[r] = y + bias[r] (QuantLinear::forward)
    uint32_t waves_per_cu;  // launch width: resident waves per compute unit; 0 = the format's default
    uint32_t rows_per_batch;  // rows a wave loads at once (1, 2 or 4); 0 = chosen from the row size
    uint32_t waves_per_row;   // 1 or 4 waves share a row; 0 = chosen from the row length
    // Further matrices of the same format and row length sharing A (q/k/v, gate/up): n_mats - 1
    // entries, each with its own output vector, bias and row count (0 = n_rows).
    uint32_t n_mats = 1;
    const uint8_t *W_more[3] = {nullptr, nullptr, nullptr};
    float *out_more[3] = {nullptr, nullptr, nullptr};
    const float *bias_more[3] = {nullptr, nullptr, nullptr};
    uint32_t n_rows_more[3] = {0, 0, 0};
    // Grouped (mixture-of-experts) form for a handful of token rows: n_pairs matvecs in one launch, pair p = the
    // matrix at W + e * w_stride (e: the group whose rows group_offsets[e] .. group_offsets[e+1]-1 hold p) times
    // the activation row A + p * a_stride, into out + p * n_rows.  group_offsets: device memory, n_groups + 1
    // entries, n_groups <= 64.  n_mats, the *_more fields, X and sums are not used in this form.
    const int32_t *group_offsets = nullptr;
    uint32_t n_groups = 0, n_pairs = 0;
    size_t w_stride = 0, a_stride = 0;
};

// What the calling thread launched last (kernel template, its integer parameters, grid): kept as plain fields,
// formatted only when oxq_last_launch asks.  Lets a measurement say which instantiation it timed.
struct LaunchNote {
    const char *kernel = "";
    uint32_t type = 0;
    int p[4] = {0, 0, 0, 0};
    uint32_t grid_x = 0, grid_y = 0, block = 0;
};
extern thread_local LaunchNote g_last_launch;
inline void note_launch(const char *kernel, uint32_t type, int p0, int p1, int p2, int p3, uint32_t gx, uint32_t gy,
                        uint32_t block) {
    g_last_launch = LaunchNote{kernel, type, {p0, p1, p2, p3}, gx, gy, block};
}

// Measurement: device buffer (and its size in bytes) that the timestamping GEMV instantiations write to; null = off.
extern std::atomic<uint64_t *> g_phase_buf;
extern std::atomic<size_t> g_phase_cap;

// Number of compute units of the current device (cached per device).
uint32_t device_cus();

hipError_t launch_gemv_q8(uint32_t type, const GemvArgs &a, hipStream_t stream);
// QuantKernel::gemv as the reference computes it (fp32 activations, weights dequantized in registers):
// out[r] = (old ? old[r] : 0) + W[r, :] . x.  hipErrorNotSupported: no such kernel for this format.
hipError_t launch_gemv_f32(uint32_t type, const uint8_t *W, const float *x, float *out, const float *old,
                           uint32_t n_rows, uint32_t n_cols, hipStream_t stream);
bool gemv_f32_supported(uint32_t type);
// True when the GEMV of this row length can quantize fp32 activations itself (GemvArgs::X).
bool gemv_takes_f32(uint32_t type, uint32_t n_cols);

// 2..4 activation vectors against one weight matrix in one launch (a small decode batch).
struct GemvVecsArgs {
    const uint8_t *W;
    const uint8_t *A;    // vector v: Q8_0 blocks at A + v * a_stride
    size_t a_stride;     // bytes
    float *out;          // vector v: out + v * out_stride
    size_t out_stride;   // floats
    uint32_t n_vecs;     // 2, 3 or 4
    uint32_t n_rows, n_cols;
    int accumulate;
    const float *bias = nullptr;  // with accumulate == 0: added to every vector's result
};
hipError_t launch_gemv_vecs(uint32_t type, const GemvVecsArgs &a, hipStream_t stream);
// Most activation vectors one launch takes for rows of n_cols columns (4, 2, or 0: none).
uint32_t gemv_vecs_max(uint32_t type, uint32_t n_cols);
// Columns of one lane's unit (32 or 64; 0: unknown type) and weights per exact integer group sum.
uint32_t gemv_unit_cols(uint32_t type);
uint32_t gemv_group_cols(uint32_t type);
// The formats beyond the first five live in a translation unit of their own.
hipError_t launch_gemv_q8_more(uint32_t type, const GemvArgs &a, hipStream_t stream);
// ffn_gate, ffn_up, SwiGLU and the Q8_0 quantizer of h in one launch (both matrices of `type`, n_rows a
// multiple of 32).  hipErrorNotSupported: no such kernel for this type / row length.
// grp.offsets set: the grouped (mixture-of-experts) form for a handful of token rows -- row p of acts (n_pairs rows)
// against the gate and up matrices of its expert e (the group of grp.offsets that holds p), Wg + e * wg_stride and
// Wu + e * wu_stride; row p of hq / h.
struct GateUpGroups {
    const int32_t *offsets = nullptr;  // device memory, n_groups + 1 entries, n_groups <= 64; null: the dense form
    uint32_t n_groups = 0, n_pairs = 0;
    size_t wg_stride = 0, wu_stride = 0;
};
hipError_t launch_gate_up_swiglu(uint32_t type, const uint8_t *Wg, const uint8_t *Wu, const uint8_t *acts, uint8_t *hq,
                                 float *h, uint32_t n_rows, uint32_t n_cols, hipStream_t stream,
                                 const GateUpGroups &grp = GateUpGroups());
hipError_t launch_gate_up_swiglu_more(uint32_t type, const uint8_t *Wg, const uint8_t *Wu, const uint8_t *acts,
                                      uint8_t *hq, float *h, uint32_t n_rows, uint32_t n_cols, hipStream_t stream,
                                      const GateUpGroups &grp = GateUpGroups());
hipError_t launch_gemv_vecs_more(uint32_t type, const GemvVecsArgs &a, hipStream_t stream);

// x: n floats (n % 32 == 0) -> n/32 Q8_0 blocks of 34 bytes.
hipError_t launch_quantize_q8_0(const float *x, size_t n, uint8_t *out, hipStream_t stream);

// h = silu(gate) * up over n floats (n % 32 == 0); h (fp32) and/or out (Q8_0 blocks) may be null.
hipError_t launch_swiglu_quantize(const float *gate, const float *up, size_t n, float *h, uint8_t *out,
                                  hipStream_t stream);
// RMSNorm of `rows` rows of n floats (n % 32 == 0); y (fp32) and/or out (Q8_0 blocks) may be null.
hipError_t launch_rmsnorm_quantize(const float *x, const float *weight, float eps, size_t rows, uint32_t n, float *y,
                                   uint8_t *out, hipStream_t stream);
// out += b (a x) * scale; r = rank floats of scratch.
hipError_t launch_lora_apply(const float *a, const float *b, float *r, uint32_t rank, float scale, const float *x,
                             float *out, uint32_t out_features, uint32_t in_features, hipStream_t stream);

// Mixture-of-experts glue: grouped activation rows from the tokens' fp32 inputs; weighted combine of the
// selected experts' outputs per token, in selection order.
hipError_t launch_moe_gather_quantize(const float *x, const int32_t *pair_token, uint8_t *out, size_t n_pairs,
                                      uint32_t hidden, hipStream_t stream);
hipError_t launch_moe_combine(const float *y_pairs, const int32_t *token_rows, const float *weights, float *out,
                              uint32_t n_tokens, uint32_t top_k, uint32_t hidden, hipStream_t stream,
                              uint32_t splits = 1, size_t split_stride = 0);

hipError_t launch_fill_zero(float *out, size_t n, hipStream_t stream);

// Router of the mixture-of-experts layer and the grouping of its (token, expert) pairs; k <= n_exp.
// acts_one (one token only, hidden a multiple of 32, a handful of choices): the same launch also writes the
// grouped Q8_0 activation rows there, k copies of the token's blocks, so that no gather launch is needed.
hipError_t launch_moe_route(const float *router, const float *x, int32_t *experts, float *weights, uint32_t n_tokens,
                            uint32_t n_exp, uint32_t hidden, uint32_t k, int32_t *offsets, int32_t *pair_token,
                            int32_t *token_rows, hipStream_t stream, uint8_t *acts_one = nullptr,
                            float *logits_scratch = nullptr);  // (room for n_tokens x n_exp floats, or null)

// The vocabulary projection and the k largest logits in one launch (oxq_lm_head.hip): bytes of workspace it needs for
// this shape (0: the one-launch form does not apply), and the launch (hipErrorNotSupported likewise).
size_t lm_head_topk_lists_bytes(uint32_t type, uint32_t n_rows, uint32_t n_cols, uint32_t k);
hipError_t launch_lm_head_topk(uint32_t type, const uint8_t *W, const uint8_t *A, float *out, uint32_t n_rows, uint32_t n_cols,
                               uint32_t k, void *lists, float *out_vals, uint32_t *out_idx, hipStream_t stream);
// Exact top-k (k <= 256, n <= 2^20) of an fp32 vector; workspace of topk_workspace_bytes(n, k) bytes (0: unsupported).
size_t topk_workspace_bytes(size_t n, size_t k);
hipError_t launch_topk(const float *x, uint32_t n, uint32_t k, float *out_vals, uint32_t *out_idx, void *workspace,
                       hipStream_t stream);
// The sampler's steps before the candidate list: banned tokens, logit bias, repetition penalty, on the logits in place.
hipError_t launch_logits_edit(float *logits, uint32_t n, const uint32_t *banned, uint32_t n_banned, const uint32_t *bias_tokens,
                              const float *bias_values, uint32_t n_bias, const uint32_t *recent, uint32_t n_window,
                              float penalty, hipStream_t stream);
// The sampler's steps after the candidate list (temperature, softmax, min-p, top-p, draw) on k <= 256 candidates.
hipError_t launch_sample_candidates(const float *vals, const uint32_t *idx, uint32_t k, float temperature, float min_p,
                                    float top_p, uint64_t *rng_state, uint32_t *token_out, float *probs_out,
                                    hipStream_t stream);

struct GemmArgs {
    const uint8_t *W;   // raw GGUF blocks [n x k]
    const uint8_t *A;   // Q8_0 blocks of the m activation rows, row-major, k/32 blocks per row
    float *out;         // [m x n] row-major
    int32_t *sums;      // optional debug dump [m][n][k/32]
    bool scaled_sums = false;  // the dump is the prefill kernel's: sub-block scale times integer sum (exact integers)
    uint8_t *workspace; // gemm_workspace_bytes(m, k) bytes, 256-byte aligned; null: row-by-row matvecs
    size_t workspace_bytes = 0;  // what the workspace really holds, if known: gemm_workspace_bytes(m, k, n, type)
                                 // bytes leave room for the few-token kernel's split-k sums
    bool by_rows = false;  // plain matmul: take the GEMV launches even though a workspace is there (the caller's
                           // snapshot of gemm_uses_tiles, so that one call reads the tuning knobs once)
    uint32_t m, n, k;   // m = all token rows (of all experts in the grouped form)
    int accumulate;
    const float *bias = nullptr;  // with accumulate == 0: out[t][r] = y + bias[r] (QuantLinear::forward_batch)
    // Grouped (mixture-of-experts) form: expert e multiplies token rows offsets[e] ..
    // offsets[e+1]-1 by the weights at W + e * w_stride.  offsets == null: plain matmul.
    const int32_t *offsets = nullptr;  // device memory, n_experts + 1 entries
    uint32_t n_experts = 0;
    uint32_t max_rows = 0;             // upper bound of the rows of any one expert (sizes the grid)
    uint32_t shape_rows = 0;           // rows per expert the tile shape is chosen for (<= max_rows)
    // Tile kernel, calls in a row on the same activations and workspace (gate then up): what the workspace holds.
    // A call that runs the re-layout pass records it here; a later call whose format needs the same byte order
    // (and no plane the earlier pass left out) skips its own pass.  Calls served by a kernel that reads the
    // caller's Q8_0 rows itself leave the record as it is.  Null: always re-lay out.
    struct Prepared {
        bool valid = false;
        int perm = 0;      // byte order of the activation payload
        bool p16 = false;  // the half-block planes of P were written as well
    };
    Prepared *prep_state = nullptr;
    size_t w_stride = 0;
    // Grouped form whose caller adds the per-split sums itself (the mixture-of-experts layer's combine launch):
    // where the few-token kernel splits k it then leaves `out` untouched, skips its reduction launch and reports
    // the sums ([splits][m][n] floats) and their count here.  Null: the call always finishes `out`.
    struct SplitSums {
        const float *partial = nullptr;
        uint32_t splits = 0;
    };
    SplitSums *defer_reduce = nullptr;
};
hipError_t launch_gemm_q8(uint32_t type, const GemmArgs &a, hipStream_t stream);
// Device scratch the tile kernel needs for m tokens of k columns (activation re-layout).
// With n and the format: plus, for a matmul of at most 32 token rows that the few-token kernel would split over k,
// the room for its per-split sums (behind the re-tiled activations, 256-byte aligned).
size_t gemm_workspace_bytes(uint32_t m, uint32_t k, uint32_t n = 0, uint32_t type = 0);
// ... of the grouped form: the planes, plus room for two per-split sums of [m x n] where the few-token kernel may
// split an expert's k in two (Q4_K / IQ4_XS, k a multiple of 1024, at most 8192 rows per expert).
size_t gemm_grouped_workspace_bytes(uint32_t m, uint32_t k, uint32_t n, uint32_t type);
// The prefill kernel of the formats whose scaled weights are exact in f16 (oxq_gemm_prefill.hip): plain matmuls of
// many token rows.  Its workspace (f16 token operands, scale pairs, bf16 pieces of the block sums) replaces the tile
// kernel's planes at the head of the caller's workspace.  hipErrorNotSupported: not this format / shape.
bool gemm_prefill_supported(uint32_t type, uint32_t m, uint32_t n, uint32_t k);
size_t gemm_prefill_workspace_bytes(uint32_t m, uint32_t k);
hipError_t launch_gemm_prefill(uint32_t type, const GemmArgs &a, hipStream_t stream);
// Tuning knobs (oxq_tuning.h), read once per call.
extern std::atomic<int> g_gemm_variant;              // 0 = default tile shape
extern std::atomic<uint32_t> g_gemm_tile_min_rows;   // 0 = default threshold
// True when (type, m, k) is served by the int8-MFMA tile kernel.
bool gemm_uses_tiles(uint32_t type, uint32_t m, uint32_t n, uint32_t k);
// Grouped (mixture-of-experts) matmuls of at most this many token rows in all take one GEMV launch, a matvec per row.
constexpr uint32_t GROUPED_GEMV_MAX_ROWS = 8;
// ... and with many experts up to half as many rows as experts: most rows then have an expert to themselves, and the
// few-token kernel, which reads a matrix once however many rows share it, has little to share (128 experts of
// 768 x 2048, top-8, the layer at 2 / 4 tokens: 40 / 50 us against 69 / 76 on the few-token kernel).
inline uint32_t grouped_gemv_max_rows(size_t n_experts) {
    const size_t q = n_experts / 2;
    return q > GROUPED_GEMV_MAX_ROWS ? (uint32_t)(q > 65535 ? 65535 : q) : GROUPED_GEMV_MAX_ROWS;
}
// Below gemm_uses_tiles' row threshold, but the few-token kernel (k split over work groups) still beats the GEMV
// launches: for callers that hold a workspace of gemm_workspace_bytes(m, k, n, type).
bool gemm_few_rows_pay(uint32_t type, uint32_t m, uint32_t n, uint32_t k);
// True when the tile kernel can take (type, m, k) at all (the grouped form always uses it).
bool gemm_tiles_supported(uint32_t type, uint32_t m, uint32_t k);

}  // namespace oxq
