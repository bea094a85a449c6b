/*
 * oxq.h -- C ABI of liboxq_hip.so: oxillama-quant's quantized matmul hot path on
 * one MI355X (gfx950), hand-written HIP.
 *
 * The entry points are what an `impl QuantKernel for HipKernel` in the reference
 * crate would bind over `extern "C"`: plain pointers and sizes, an int status per
 * call, nothing retained beyond the call unless a handle says so.  Citations name
 * the reference interface each one stands in for (paths relative to the reference
 * tree, Q/ = crates/oxillama-quant/src).
 *
 * Weight bytes are raw GGUF blocks exactly as `GgufModel::tensor_data` hands them
 * out (crates/oxillama-gguf/src/loader.rs:115), row-major, row_bytes =
 * ceil(n_cols / block_size) * block_bytes (Q/reference/q4_k.rs:130-131).  They go
 * to HBM unchanged; nothing is repacked.
 *
 * Rows that end inside a block (n_cols not a multiple of the block size): the
 * matvec, gemv and gemm entry points, on host slices and on device pointers, skip
 * the columns past n_cols as the reference's kernels do (Q/reference/q4_k.rs:307-321,
 * Q/traits.rs:150-166) -- whole blocks are stored and read, whole Q8_0 activation
 * blocks are expected (their bytes past n_cols are ignored).  The fused layers
 * (feed-forward, mixture of experts, QuantLinear on device pointers), the grouped
 * matmul, the GGUF loader and the debug dumps of the group sums take whole blocks
 * only and return OXQ_ERR_UNSUPPORTED_SHAPE otherwise, so that the caller can fall
 * back to its CPU kernel.
 *
 * Thread safety: every function may be called from several host threads; calls
 * taking host slices serialise on an internal lock.  Calls on device pointers are
 * asynchronous on the caller's stream, with two documented exceptions that
 * synchronise that stream and therefore cannot be recorded into a HIP graph: the
 * forms of oxq_gemm_q8_dev and oxq_block_sums_dev that are given no workspace.
 *
 * Every entry point below cites the reference interface it stands in for.  The
 * launch-shape knobs used for measurement live in oxq_tuning.h and are not part of
 * what the reference-side shim binds.
 */
#ifndef OXQ_H
#define OXQ_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* GgufTensorType discriminants, crates/oxillama-gguf/src/types.rs:72-150. */
#define OXQ_TYPE_Q4_0 2u
#define OXQ_TYPE_Q8_0 8u
#define OXQ_TYPE_Q4_K 12u
#define OXQ_TYPE_Q6_K 14u
#define OXQ_TYPE_IQ4_XS 23u
/* Further formats: GEMV and dequant_block for all of them; the int8-MFMA tile kernel (prefill, expert
 * groups) for Q4_1, Q5_0, Q5_1, Q8_1, Q5_K, IQ4_NL; Q2_K and Q3_K run the batched form by rows. */
#define OXQ_TYPE_Q4_1 3u
#define OXQ_TYPE_Q5_0 6u
#define OXQ_TYPE_Q5_1 7u
#define OXQ_TYPE_Q8_1 9u
#define OXQ_TYPE_Q2_K 10u
#define OXQ_TYPE_Q3_K 11u
#define OXQ_TYPE_Q5_K 13u
#define OXQ_TYPE_IQ4_NL 20u

/* Status codes: 1..7 are the QuantError variants of Q/error.rs:10-71 in order;
 * the (expected, got) / (needed, available) pair of the failing check is kept per
 * thread and read back with oxq_last_error(). */
#define OXQ_OK 0
#define OXQ_ERR_UNSUPPORTED_TYPE 1     /* QuantError::UnsupportedType */
#define OXQ_ERR_BLOCK_SIZE_MISMATCH 2  /* QuantError::BlockSizeMismatch */
#define OXQ_ERR_DIMENSION_MISMATCH 3   /* QuantError::DimensionMismatch{expected, got} */
#define OXQ_ERR_KERNEL 4               /* QuantError::KernelError{message} (HIP failures) */
#define OXQ_ERR_BLOCK_COUNT_MISMATCH 5 /* QuantError::BlockCountMismatch */
#define OXQ_ERR_BUFFER_TOO_SMALL 6     /* QuantError::BufferTooSmall{needed, available} */
#define OXQ_ERR_INTERNAL 7             /* QuantError::Internal{message} */
#define OXQ_ERR_UNSUPPORTED_SHAPE 8    /* no reference counterpart: fall back to the CPU kernel */
#define OXQ_ERR_NO_DEVICE 9            /* no reference counterpart: no usable GPU */

typedef struct oxq_device_props {
    int device;
    int compute_units;
    int clock_khz;        /* peak engine clock */
    int memory_clock_khz;
    int memory_bus_bits;
    size_t total_memory;
    char name[128];
    char arch[64];
} oxq_device_props;

/* Opaque handle to weights resident in HBM. */
typedef struct oxq_weights *oxq_weights_t;

/* ---- lifetime ---------------------------------------------------------- */

/* Select the GPU used by this library (KernelDispatcher::new + SimdCapabilities::
 * detect, Q/dispatch.rs:42,131: the run-time capability probe of the tier).
 * Idempotent.  OXQ_ERR_NO_DEVICE when no gfx950-class device is visible. */
int oxq_init(int device);
/* Free cached weights and scratch memory.  Handles become invalid. */
int oxq_shutdown(void);
int oxq_device_info(oxq_device_props *out);

/* Detail of the last failing call on this thread.  `a` = expected / needed,
 * `b` = got / available; `message` may be NULL. */
int oxq_last_error(size_t *a, size_t *b, char *message, size_t message_len);
const char *oxq_status_name(int status);

/* ---- format metadata: QuantKernel::block_size / block_bytes / name ----- */
/* Q/traits.rs:175-182; values of crates/oxillama-gguf/src/types.rs:199-262.  0 /
 * NULL for a format this library has no kernel for. */
size_t oxq_block_size(uint32_t type);
size_t oxq_block_bytes(uint32_t type);
const char *oxq_type_name(uint32_t type);
/* KernelDispatcher::get_kernel, Q/dispatch.rs:141: OXQ_OK if a HIP kernel exists
 * for `type`, else OXQ_ERR_UNSUPPORTED_TYPE (the shim then tries the next tier). */
int oxq_get_kernel(uint32_t type);

/* ---- QuantKernel methods on host slices (the drop-in route) ------------ */

/* QuantKernel::dequant_block, Q/traits.rs:28.  Checks as Q/reference/q4_k.rs:
 * 53-64: block_len < block_bytes -> BUFFER_TOO_SMALL, then out_len < block_size
 * -> BUFFER_TOO_SMALL.  Runs on the GPU. */
int oxq_dequant_block(uint32_t type, const uint8_t *block, size_t block_len, float *output,
                      size_t output_len);

/* quantize_f32_to_q8_0, Q/quantize.rs:58-75.  n % 32 != 0 -> DIMENSION_MISMATCH
 * {expected: (n/32+1)*32, got: n}.  out_len must hold n/32 * 34 bytes.  Output
 * bytes are bit-identical to the reference encoder (Q/quantize.rs:190-210). */
int oxq_quantize_f32_to_q8_0(const float *data, size_t n, uint8_t *out, size_t out_len);

/* QuantKernel::matvec_q8_fused, Q/traits.rs:89-96: out[r] += W[r,:] . acts
 * (ACCUMULATE).  Validation order of Q/reference/q4_k.rs:226-250: out_len <
 * n_rows -> DIMENSION_MISMATCH{n_rows, out_len}; weights_len < n_rows*row_bytes
 * -> BUFFER_TOO_SMALL; acts_len < blocks_per_row*(block_size/32)*34 ->
 * BUFFER_TOO_SMALL. */
int oxq_matvec_q8_fused(uint32_t type, const uint8_t *weights, size_t weights_len,
                        const uint8_t *acts_q8, size_t acts_len, float *out, size_t out_len,
                        size_t n_rows, size_t n_cols);

/* QuantKernel::gemv, Q/traits.rs:39-44, on a QuantTensor given as (data, shape,
 * type) (Q/types.rs:11-18).  output[r] is overwritten.  n_rows = shape[0], n_cols
 * = shape[1] (or n_elements / n_rows for a 1-d shape), Q/reference/q4_k.rs:110-115;
 * input_len < n_cols -> DIMENSION_MISMATCH{n_cols, input_len}; output_len <
 * n_rows -> DIMENSION_MISMATCH{n_rows, output_len} (:117-128).
 * The activation vector is quantized to Q8_0 on the GPU and fed to the fused
 * kernel: results equal oxq_quantize_f32_to_q8_0 + oxq_matvec_q8_fused into
 * zeros, and differ from the reference's f32-activation gemv by the Q8_0
 * rounding of the input.  Where n_cols is not a multiple of the block size the
 * input is taken as zero-padded to whole blocks (the reference's gemv skips those
 * columns, Q/reference/q4_k.rs:161,168). */
int oxq_gemv(uint32_t type, const uint8_t *data, size_t data_len, const size_t *shape,
             size_t n_dims, const float *input, size_t input_len, float *output,
             size_t output_len);

/* QuantKernel::gemm, Q/traits.rs:58-66: input [m x k] row-major, output [m x n]
 * row-major, overwritten; same activation handling as oxq_gemv, row by row
 * (Q/reference/q4_k.rs:186-201). */
int oxq_gemm(uint32_t type, const uint8_t *data, size_t data_len, const size_t *shape,
             size_t n_dims, const float *input, size_t input_len, float *output,
             size_t output_len, size_t m, size_t n, size_t k);

/* Debug: exact int32 group sums of the fused kernel, sums[r * groups + g] with
 * groups = n_cols/32 (n_cols/16 for Q6_K).  Q4_0: sum (q-8)a; Q8_0: sum w a;
 * Q4_K: sum q a; Q6_K: sum (q-32)a; IQ4_XS: sum kvalues[q] a.  No reference
 * counterpart (the reference's AVX2 rows form the same sums in registers,
 * Q/simd/avx2/q4_k.rs:298-318). */
int oxq_block_sums(uint32_t type, const uint8_t *weights, size_t weights_len,
                   const uint8_t *acts_q8, size_t acts_len, int32_t *sums, size_t sums_len,
                   size_t n_rows, size_t n_cols);

/* Host-slice calls can keep a device copy of each weight buffer, keyed by (pointer,
 * length, type), so that repeated calls with the same QuantTensor do not cross PCIe
 * again.  Stands in for the ownership the reference gets for free from host slices
 * (Q/types.rs:11-18: QuantTensor.data is an owned, immutable Vec<u8> after load).
 * Off by default.  The contract of mode 1: while a buffer is cached the caller does
 * not change its bytes and does not free it -- or calls oxq_weight_cache_invalidate
 * with its address first (a freed address that the allocator hands out again with
 * other weights would otherwise hit the old copy).  Mode 1 guards that contract only
 * loosely, with a fingerprint of 64 sampled 64-byte pieces; mode 2 hashes every byte
 * of the buffer on every call, so that any change is seen and the buffer uploaded
 * again (slower than the upload it saves on PCIe 5: for checking a caller against the
 * contract, not for production).  Resident handles (oxq_weights_register) are the
 * route without any of this.  The cache holds at most oxq_weight_cache_set_limit
 * bytes (default 16 GiB; least recently used copies are freed first; a buffer larger
 * than the limit is staged per call as if the cache were off). */
int oxq_weight_cache_enable(int mode); /* 0 off, 1 on, 2 on and verified */
int oxq_weight_cache_clear(void);
int oxq_weight_cache_invalidate(const void *host_ptr);
int oxq_weight_cache_set_limit(size_t max_bytes);
/* entries, bytes held, hits and uploads since the library was loaded (any may be null). */
int oxq_weight_cache_stats(size_t *entries, size_t *bytes, uint64_t *hits, uint64_t *uploads);

/* ---- weights resident in HBM ------------------------------------------- */

/* Copy a weight matrix to HBM once (what load_quant_linear's data.to_vec() is to
 * the CPU path, crates/oxillama-arch/src/llama/model.rs:805-822). */
int oxq_weights_register(uint32_t type, size_t n_rows, size_t n_cols, const uint8_t *bytes,
                         size_t len, oxq_weights_t *handle);
int oxq_weights_release(oxq_weights_t handle);
/* Device address / byte length of the registered blocks. */
void *oxq_weights_device_ptr(oxq_weights_t handle);
size_t oxq_weights_nbytes(oxq_weights_t handle);

/* ---- device-pointer entry points (no copies, asynchronous) ------------- */
/* All pointers are device memory; `stream` is a hipStream_t (NULL = default
 * stream).  Shapes are validated as above (lengths are the caller's promise);
 * kernels are enqueued and the call returns.  Q6_K weight matrices must start on
 * a 4-byte boundary (device allocations and GGUF tensor data do); OXQ_ERR_KERNEL
 * otherwise. */

/* quantize_f32_to_q8_0 over `rows` rows of n floats each (rows*n contiguous). */
int oxq_quantize_q8_0_dev(const float *d_x, size_t n_total, uint8_t *d_out, void *stream);

/* matvec_q8_fused: d_out[r] += ... ; accumulate = 0 overwrites instead (gemv). */
int oxq_matvec_q8_fused_dev(uint32_t type, const uint8_t *d_weights, const uint8_t *d_acts_q8,
                            float *d_out, size_t n_rows, size_t n_cols, int accumulate,
                            void *stream);

/* The same for up to 4 weight matrices of one format and shape that share the activation
 * vector -- wq/wk/wv or ffn_gate/ffn_up of one layer, which the reference runs as separate
 * QuantLinear::forward calls on the same input (crates/oxillama-arch/src/llama/model.rs:
 * 295-310): d_outs[i][r] (+)= d_weights[i][r,:] . acts.  One launch streams all of them, which
 * saves the fill and drain of the memory pipeline between them.  d_weights / d_outs are host
 * arrays of n_mats device pointers.  Results are bit-identical to n_mats single calls. */
int oxq_matvec_q8_fused_multi_dev(uint32_t type, size_t n_mats, const uint8_t *const *d_weights,
                                  const uint8_t *d_acts_q8, float *const *d_outs, size_t n_rows,
                                  size_t n_cols, int accumulate, void *stream);

/* QuantKernel::gemv on device pointers (Q/traits.rs:39-44: fp32 input): d_out[r] (+)= W[r,:] . q8(x).
 * Every work group of the kernel first quantizes d_x (n_cols floats) to Q8_0 into LDS with the
 * reference encoder's arithmetic, so the result is bit-identical to oxq_quantize_q8_0_dev + oxq_matvec_q8_fused_dev
 * at one launch instead of two.  oxq_gemv_multi_dev: the same for up to 4 matrices of one shape
 * and format sharing x.  Rows of more than 46080 columns (the quantized vector is staged in
 * LDS) return OXQ_ERR_UNSUPPORTED_SHAPE: quantize first. */
int oxq_gemv_dev(uint32_t type, const uint8_t *d_weights, const float *d_x, float *d_out,
                 size_t n_rows, size_t n_cols, int accumulate, void *stream);
int oxq_gemv_multi_dev(uint32_t type, size_t n_mats, const uint8_t *const *d_weights,
                       const float *d_x, float *const *d_outs, size_t n_rows, size_t n_cols,
                       int accumulate, void *stream);

/* QuantKernel::gemv with the reference's own numerics (Q/traits.rs:39-44; rows: Q/reference/q4_0.rs:82-102,
 * q8_0.rs:77-92, q4_k.rs:135-178, q6_k.rs:108-166, iq4_xs.rs:130-163; what QuantLinear::forward calls,
 * crates/oxillama-arch/src/common/linear.rs:77-98): the fp32 activations are NOT quantized; every weight is
 * dequantized in registers and every term is formed by the reference's scalar expression, in its column order
 * inside a block; the reference's running sum over the row becomes a tree over lanes and waves, which moves the
 * result by rounding only (within 1e-5 of |y|inf of the reference gemv).  d_out[r] = W[r,:] . x (+ d_bias[r] when
 * d_bias is given; + d_out[r] when accumulate is set; not both).  n_cols need not be a block multiple (columns
 * past it are skipped, as in the reference).  Formats: Q4_0, Q8_0, Q4_K, Q6_K, IQ4_XS; others return
 * OXQ_ERR_UNSUPPORTED_TYPE.  About twice the time of the Q8_0-activation route at decode shapes. */
int oxq_gemv_f32_dev(uint32_t type, const uint8_t *d_weights, const float *d_x, const float *d_bias,
                     float *d_out, size_t n_rows, size_t n_cols, int accumulate, void *stream);

/* Which arithmetic the entry points that take fp32 input and mirror QuantKernel::gemv / gemm and
 * QuantLinear::forward / forward_batch use (oxq_gemv, oxq_gemm, oxq_linear_forward, oxq_linear_forward_batch,
 * and oxq_linear_forward_dev when it is given no Q8_0 activations):
 *   OXQ_ROUTE_Q8  (default) x is quantized to Q8_0 and the fused kernels run -- the reference's
 *                 matvec_q8_fused arithmetic, the fast route;
 *   OXQ_ROUTE_F32 the reference's gemv arithmetic (oxq_gemv_f32_dev); formats without such a kernel
 *                 then return OXQ_ERR_UNSUPPORTED_TYPE instead of changing arithmetic silently.
 * Process-wide, atomic; takes effect for calls that start afterwards. */
#define OXQ_ROUTE_Q8 0
#define OXQ_ROUTE_F32 1
int oxq_select_activation_route(int route);
int oxq_activation_route(void);

/* Prefill / decode batch: d_out[m x n] (+)= acts[m rows of Q8_0] x W[n x k]^T, the batched
 * form of matvec_q8_fused (m fused matvecs, Q/reference/q4_k.rs:186-201).  From 5 rows up
 * (6 where n < 8192, 9 on matrices of fewer than 2^24 weights), with k a multiple of 256 and at
 * most 65536 (the formats of 32-weight blocks: any multiple of 32 from 256 up), every format runs
 * on the int8-MFMA tile
 * kernel, which needs oxq_gemm_q8_workspace_bytes() bytes of 256-byte-aligned device scratch:
 * pass it and the call is asynchronous and allocation-free; pass NULL and the library uses
 * its own scratch (the call then serialises and waits for the stream).  Fewer rows, and
 * shapes for which the workspace size is 0, run GEMV launches (up to four rows per pass over
 * the weights) and ignore the workspace.  Decode batches (3..16 rows, up to 32 on matrices of
 * fewer than 8192 rows) in every weight format but Q8_1 run on a kernel that
 * reads the weights once and splits k over work groups; its per-split sums are part of the
 * workspace size.  Q4_K matmuls of many token rows whose 128-token x
 * 256-row work groups fill the chip (the prefill shapes) run on the f16 matrix cores instead,
 * with the 6-bit sub-block scale inside the weight operand (exact) and d / dmin applied per
 * super-block: the same integers, fp32 inside the same 1e-5 bar; the workspace size covers both. */
size_t oxq_gemm_q8_workspace_bytes(uint32_t type, size_t m, size_t n, size_t k);
int oxq_gemm_q8_dev(uint32_t type, const uint8_t *d_weights, const uint8_t *d_acts_q8,
                    float *d_out, size_t m, size_t n, size_t k, int accumulate,
                    void *d_workspace, size_t workspace_bytes, void *stream);
/* oxq_gemm_q8_dev for callers that cannot allocate device memory and have no workspace to pass
 * (code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc).  No
 * counterpart in the reference.  The tile kernel's workspace is a static array in device
 * memory that the library holds on each GPU it was initialised on (16 MiB:
 * oxq_gemm_q8_static_max_workspace_bytes()); the call allocates nothing, synchronises nothing and
 * gives the bits of oxq_gemm_q8_dev.  Shapes whose oxq_gemm_q8_workspace_bytes exceeds the
 * array return OXQ_ERR_BUFFER_TOO_SMALL (needed, available); oxq_init must have run (the call
 * does not initialise lazily: OXQ_ERR_NO_DEVICE) for the device the calling thread has current,
 * whose copy of the array the call uses.  All calls on one GPU share the array: issue them on
 * ONE stream per GPU (or order the streams with events yourself) -- calls that overlap in time
 * on one GPU race on it, and nothing in the library detects that. */
size_t oxq_gemm_q8_static_max_workspace_bytes(void);
int oxq_gemm_q8_static_dev(uint32_t type, const uint8_t *d_weights, const uint8_t *d_acts_q8,
                           float *d_out, size_t m, size_t n, size_t k, int accumulate,
                           void *stream);
/* Debug: as oxq_gemm_q8_dev (overwrite), and the exact int32 group sums of the tile
 * kernel, d_sums[(r * n + c) * groups + g], groups = k/32 (k/16 for Q6_K).  For Q4_0 the
 * (and Q5_0) the tile kernel multiplies the unsigned values (sum q*a); the "- 8" ("- 16") enters in
 * fp32.  OXQ_ERR_UNSUPPORTED_SHAPE when the shape has no tile kernel. */
int oxq_gemm_block_sums_dev(uint32_t type, const uint8_t *d_weights, const uint8_t *d_acts_q8,
                            float *d_out, int32_t *d_sums, size_t m, size_t n, size_t k,
                            void *d_workspace, size_t workspace_bytes, void *stream);
/* Debug: the same for the prefill kernel of the formats whose scaled weights are exact in f16 (Q4_K), which
 * oxq_gemm_q8_dev takes for many token rows: its matrix-core result per (token, row, 32-weight sub-block) is the
 * 6-bit sub-block scale times the integer group sum, an exact integer, written to
 * d_sums[(r * n + c) * (k/32) + g]; d_out as oxq_gemm_q8_dev (overwrite).  Any m >= 1 runs on that kernel here.
 * OXQ_ERR_UNSUPPORTED_SHAPE when the format or shape has no such kernel; a workspace is required. */
int oxq_gemm_scaled_sums_dev(uint32_t type, const uint8_t *d_weights, const uint8_t *d_acts_q8,
                             float *d_out, int32_t *d_sums, size_t m, size_t n, size_t k,
                             void *d_workspace, size_t workspace_bytes, void *stream);

/* Grouped (mixture-of-experts) matmul: the batched form of the per-token expert calls of
 * MoeFfn::forward (crates/oxillama-arch/src/common/moe.rs:236-252: for each selected expert,
 * expert.forward(input) -> QuantLinear::forward -> gemv).  Token rows are grouped by
 * expert: expert e multiplies rows d_row_offsets[e] .. d_row_offsets[e+1]-1 of d_acts_q8
 * (total_rows rows of k/32 Q8_0 blocks) by the n x k weights at d_weights + e *
 * expert_stride_bytes and writes the same rows of d_out [total_rows x n].  d_row_offsets is
 * device memory (n_experts + 1 ascending int32 values, last = total_rows), so the call neither
 * copies nor synchronises; max_rows_per_expert bounds any one group (0 = total_rows) and only
 * sizes the launch (which kernel and tile shape serve the call follows from it and from the mean
 * group size: fp32 summation order, hence the last bits, can differ between two bounds; every
 * choice meets the 1e-5 bar).  k must be a multiple of 256 (the formats of 32-weight blocks: of
 * 32, and at least 256); needs oxq_moe_gemm_q8_workspace_bytes() bytes of
 * 256-byte-aligned device scratch (the re-tiled activations and, for Q4_K / IQ4_XS experts of
 * at most 8192 rows, room for the sums of two halves of k).  d_sums (optional, else NULL): exact int32 group sums
 * [(row * n + c) * (k/32) + g] as in oxq_gemm_block_sums_dev. */
size_t oxq_moe_gemm_q8_workspace_bytes(uint32_t type, size_t total_rows, size_t n, size_t k);
int oxq_moe_gemm_q8_dev(uint32_t type, const uint8_t *d_weights, size_t expert_stride_bytes,
                        size_t n_experts, const uint8_t *d_acts_q8, const int32_t *d_row_offsets,
                        size_t total_rows, size_t max_rows_per_expert, float *d_out, int32_t *d_sums,
                        size_t n, size_t k, int accumulate, void *d_workspace,
                        size_t workspace_bytes, void *stream);

/* ---- the callers of the kernel trait: QuantLinear, the dense SwiGLU feed-forward, RMSNorm ----
 *
 * LoRA adapter on device memory (LoraAdapter, crates/oxillama-quant/src/lora.rs:21-35): d_a is
 * [rank x in_features], d_b is [out_features x rank], both row-major fp32; d_r is rank floats
 * of device scratch that the call overwrites. */
typedef struct oxq_lora {
    const float *d_a;
    const float *d_b;
    float *d_r;
    size_t rank;
    float scale;
} oxq_lora;

/* LoraAdapter::apply (lora.rs:83-124): d_out += d_b (d_a d_x) * scale.  NULL or rank 0: no-op. */
int oxq_lora_apply_dev(const oxq_lora *lora, const float *d_x, float *d_out, size_t out_features,
                       size_t in_features, void *stream);

/* QuantLinear::forward (crates/oxillama-arch/src/common/linear.rs:77-98): d_out = W . q8(x)
 * + bias + LoRA correction, in that order.  Activations: pass d_acts_q8 (Q8_0 blocks of x,
 * quantized once for every projection that reads x), or NULL to have the kernel quantize d_x
 * itself (as oxq_gemv_dev).  d_x is needed for the LoRA term; d_bias and lora may be NULL.
 * The bias rides in the matvec's epilogue (no extra launch); LoRA adds two small launches. */
int oxq_linear_forward_dev(uint32_t type, const uint8_t *d_weights, const float *d_x,
                           const uint8_t *d_acts_q8, const float *d_bias, const oxq_lora *lora,
                           float *d_out, size_t out_features, size_t in_features, void *stream);

/* Up to 4 QuantLinear::forward calls on the same input as one launch: wq/wk/wv, or ffn_gate/
 * ffn_up, which the reference issues one after the other
 * (crates/oxillama-arch/src/llama/model.rs:295-310).  The matrices share the format and
 * in_features; each has its own out_features[i], output and optional bias (d_biases may be
 * NULL, and so may any entry).  Results are bit-identical to separate calls. */
int oxq_linear_forward_multi_dev(uint32_t type, size_t n_mats, const uint8_t *const *d_weights,
                                 const uint8_t *d_acts_q8, const float *const *d_biases,
                                 float *const *d_outs, const size_t *out_features,
                                 size_t in_features, void *stream);

/* QuantLinear::forward_batch (linear.rs:105-132): d_out[batch x out_features] = gemm + bias
 * broadcast over the batch (no LoRA, as in the reference).  Workspace as oxq_gemm_q8_dev. */
int oxq_linear_forward_batch_dev(uint32_t type, const uint8_t *d_weights,
                                 const uint8_t *d_acts_q8, const float *d_bias, float *d_out,
                                 size_t batch, size_t out_features, size_t in_features,
                                 void *d_workspace, size_t workspace_bytes, void *stream);

/* QuantLinear::forward on host slices, staged per call like oxq_gemv (drop-in route).  bias:
 * NULL or bias_len floats (a short bias covers its own length, as the reference's zip does);
 * LoRA: NULL pointers or rank 0 for none, else lora_a_len == rank * in_features and
 * lora_b_len == out_features * rank (LoraAdapter::new, lora.rs:43-73) or
 * OXQ_ERR_DIMENSION_MISMATCH. */
int oxq_linear_forward(uint32_t type, const uint8_t *data, size_t data_len, const size_t *shape,
                       size_t n_dims, const float *bias, size_t bias_len, const float *lora_a,
                       size_t lora_a_len, const float *lora_b, size_t lora_b_len, size_t rank,
                       float scale, const float *input, size_t input_len, float *output,
                       size_t output_len);

/* QuantLinear::forward_batch on host slices (linear.rs:105-132): gemm with n = shape[0] and
 * k = shape[1], then the bias added to every row of the batch. */
int oxq_linear_forward_batch(uint32_t type, const uint8_t *data, size_t data_len, const size_t *shape,
                             size_t n_dims, const float *bias, size_t bias_len, const float *input,
                             size_t input_len, float *output, size_t output_len, size_t batch);

/* swiglu_inplace (crates/oxillama-arch/src/common/swiglu.rs:15-21) fused with the quantizer of
 * the next projection's input: h = silu(gate) * up over n_total floats (a multiple of 32),
 * sigmoid = 1 / (1 + exp(-g)), h = (g * sigmoid) * u.  d_h (fp32 h) and d_out_q8 (Q8_0 blocks
 * of h, bit-exact to quantizing d_h) are each optional (NULL). */
int oxq_swiglu_quantize_q8_0_dev(const float *d_gate, const float *d_up, size_t n_total,
                                 float *d_h, uint8_t *d_out_q8, void *stream);

/* RmsNorm::forward_to (crates/oxillama-arch/src/common/rms_norm.rs:49-66) fused with the
 * quantizer: per row of n floats (a multiple of 32), y = (x * (1 / sqrt(mean(x^2) + eps))) *
 * weight.  d_y (fp32) and d_out_q8 (Q8_0 blocks of y, bit-exact to quantizing d_y) are each
 * optional (NULL).  The sum of squares is a tree sum (the reference adds in index order). */
int oxq_rmsnorm_quantize_q8_0_dev(const float *d_x, const float *d_weight, float eps, size_t rows,
                                  size_t n, float *d_y, uint8_t *d_out_q8, void *stream);

/* Dense feed-forward block (crates/oxillama-arch/src/llama/model.rs:277-310): d_out =
 * down(silu(gate(x)) * up(x)) for one token, from the Q8_0 blocks of the normed hidden state.
 * Three launches when gate and up share a format (gate + up, SwiGLU + quantize, down), four
 * otherwise.  Needs oxq_ffn_workspace_bytes() bytes of 256-byte-aligned device scratch;
 * allocates nothing and does not synchronise. */
/* ffn_gate and ffn_up (both of `type`, [intermediate x hidden]) on one Q8_0 input, SwiGLU and the
 * Q8_0 quantizer of the down projection's input in ONE launch: a work group owns 32 rows of both
 * matrices, i.e. one block of h.  d_out_q8: intermediate / 32 * 34 bytes; d_h (optional): h in
 * fp32.  The sums are those of oxq_matvec_q8_fused_dev bit for bit, so the bytes equal those of
 * the separate calls.  UnsupportedShape when the type / row length has no such kernel (rows
 * longer than 128 units, Q8_1 / IQ4_NL / Q2_K / Q3_K): use the separate calls.
 * oxq_ffn_swiglu_dev takes this route by itself when gate and up share a type. */
int oxq_ffn_gate_up_swiglu_q8_dev(uint32_t type, const uint8_t *d_gate, const uint8_t *d_up,
                                  const uint8_t *d_acts_q8, float *d_h, uint8_t *d_out_q8,
                                  size_t intermediate, size_t hidden, void *stream);
size_t oxq_ffn_workspace_bytes(size_t hidden, size_t intermediate);
int oxq_ffn_swiglu_dev(uint32_t gate_type, const uint8_t *d_gate, uint32_t up_type,
                       const uint8_t *d_up, uint32_t down_type, const uint8_t *d_down,
                       const uint8_t *d_acts_q8, float *d_out, size_t hidden, size_t intermediate,
                       void *d_workspace, size_t workspace_bytes, void *stream);

/* MoeFfn::forward (crates/oxillama-arch/src/common/moe.rs:184-258) for n_tokens tokens at once, the
 * experts' gate / up / down matrices in quantized formats (one format per projection, as in
 * oxq_ffn_swiglu_dev).
 *
 * oxq_moe_route_dev: steps 1-4 (moe.rs:189-250) for every token and the grouping of the (token,
 * expert) pairs by expert.  Logits of the fp32 router [n_experts x hidden] against d_x [n_tokens
 * x hidden], stable softmax, the k = min(top_k, n_experts) experts of largest weight in
 * descending order (the lower index first among equal weights, which the reference's
 * sort_unstable_by leaves open), weights renormalised over the selected ones.  Outputs:
 * d_experts, d_weights [n_tokens x k]; d_row_offsets [n_experts + 1] (grouped rows of expert e:
 * offsets[e] .. offsets[e+1]-1); d_pair_token [n_tokens * k] (the token of grouped row r);
 * d_token_rows [n_tokens x k] (the grouped row of each token's j-th choice).  Rows of an expert
 * are in ascending (token, choice) order: the tables do not depend on scheduling.  top_k == 0
 * is KernelError (the reference's InvalidConfig, moe.rs:168-172); at most 1024 experts.
 *
 * oxq_moe_gather_quantize_q8_0_dev: grouped activation row r = the Q8_0 blocks of
 * d_x[d_pair_token[r]] (every selected expert reads the token's own input, moe.rs:252).
 *
 * oxq_moe_combine_dev: d_out[t] = sum over j < top_k, in that order from 0.0, of d_weights[t][j]
 * * d_y_pairs[d_token_rows[t][j]] (moe.rs:240-256: product and sum rounded separately).
 *
 * oxq_moe_ffn_dev: the whole layer after routing -- gather + quantize, grouped gate and up
 * matmuls (oxq_moe_gemm_q8_dev), SwiGLU + quantize, grouped down matmul, combine.  top_k is the
 * width of the tables (the clamped k); max_rows_per_expert as in oxq_moe_gemm_q8_dev (0:
 * unknown, e.g. tables made on the device).  Expert e's matrices sit at d_gate + e *
 * gate_stride_bytes, etc.  No allocation, no synchronisation; needs
 * oxq_moe_ffn_workspace_bytes() bytes of 256-byte-aligned scratch (0: no grouped kernel for a
 * type / shape). */
int oxq_moe_route_dev(const float *d_router, const float *d_x, size_t n_tokens, size_t n_experts,
                      size_t hidden, size_t top_k, int32_t *d_experts, float *d_weights,
                      int32_t *d_row_offsets, int32_t *d_pair_token, int32_t *d_token_rows,
                      void *stream);
int oxq_moe_gather_quantize_q8_0_dev(const float *d_x, const int32_t *d_pair_token, size_t n_pairs,
                                     size_t hidden, uint8_t *d_out_q8, void *stream);
int oxq_moe_combine_dev(const float *d_y_pairs, const int32_t *d_token_rows, const float *d_weights,
                        size_t n_tokens, size_t top_k, size_t hidden, float *d_out, void *stream);
size_t oxq_moe_ffn_workspace_bytes(uint32_t gate_type, uint32_t up_type, uint32_t down_type,
                                   size_t n_pairs, size_t hidden, size_t intermediate);
int oxq_moe_ffn_dev(uint32_t gate_type, const uint8_t *d_gate, size_t gate_stride_bytes,
                    uint32_t up_type, const uint8_t *d_up, size_t up_stride_bytes,
                    uint32_t down_type, const uint8_t *d_down, size_t down_stride_bytes,
                    size_t n_experts, const float *d_x, size_t n_tokens, size_t top_k,
                    const int32_t *d_row_offsets, const int32_t *d_pair_token,
                    const int32_t *d_token_rows, const float *d_weights,
                    size_t max_rows_per_expert, float *d_out, size_t hidden, size_t intermediate,
                    void *d_workspace, size_t workspace_bytes, void *stream);

/* MoeFfn::forward (crates/oxillama-arch/src/common/moe.rs:184-258) on device pointers, for
 * n_tokens input vectors at once: oxq_moe_route_dev + oxq_moe_ffn_dev in one call, with the
 * routing tables kept in the workspace.  d_router fp32 [n_experts x hidden]; d_x, d_out fp32
 * [n_tokens x hidden]; expert e's matrices at d_gate + e * gate_stride_bytes, etc.  top_k == 0
 * is KernelError (moe.rs:168-172), top_k above n_experts is clamped (moe.rs:233); no expert or
 * intermediate == 0 gives the zeroed output (moe.rs:240-242).  The same bits as the two calls.
 * For one token (the reference's own call) the router's launch also groups the choices and
 * writes the quantized activation rows, so the layer is four launches plus the combine.  No
 * allocation, no synchronisation; needs oxq_moe_forward_workspace_bytes() bytes of 256-byte-
 * aligned scratch (0: no grouped kernel for a type / shape).  After the call the workspace
 * starts with the routing tables of oxq_moe_route_dev, each rounded up to 256 bytes: experts
 * [n_tokens x k] int32 | weights [n_tokens x k] fp32 | row offsets [n_experts + 1] int32 |
 * pair_token [n_tokens * k] int32 | token_rows [n_tokens x k] int32 (k = min(top_k, n_experts)). */
size_t oxq_moe_forward_workspace_bytes(uint32_t gate_type, uint32_t up_type, uint32_t down_type,
                                       size_t n_tokens, size_t top_k, size_t n_experts,
                                       size_t hidden, size_t intermediate);
int oxq_moe_forward_dev(uint32_t gate_type, const uint8_t *d_gate, size_t gate_stride_bytes,
                        uint32_t up_type, const uint8_t *d_up, size_t up_stride_bytes,
                        uint32_t down_type, const uint8_t *d_down, size_t down_stride_bytes,
                        size_t n_experts, const float *d_router, const float *d_x, size_t n_tokens,
                        size_t top_k, float *d_out, size_t hidden, size_t intermediate,
                        void *d_workspace, size_t workspace_bytes, void *stream);

/* MoeFfn::forward on host slices, for n_tokens input vectors at once (n_tokens = 1 is the
 * reference's call): experts' matrices as raw blocks, expert after expert (gate_len = n_experts *
 * bytes of one [intermediate x hidden] matrix, etc.), fp32 router [n_experts x hidden].  Checks
 * in the reference's order (moe.rs:151-173: router size, top_k; moe.rs:33-58: gate, up, down
 * sizes) as DimensionMismatch {expected, got} / KernelError; hidden and intermediate must be
 * multiples of 256, or of 32 from 256 up where the matrices they are the row length of are in
 * formats of 32-weight blocks (UnsupportedShape otherwise).  Stages everything to the device (weights
 * through the weight cache when it is on), runs oxq_moe_forward_dev, copies the output back. */
int oxq_moe_forward(uint32_t gate_type, const uint8_t *gate, size_t gate_len, uint32_t up_type,
                    const uint8_t *up, size_t up_len, uint32_t down_type, const uint8_t *down,
                    size_t down_len, const float *router, size_t router_len, size_t n_experts,
                    size_t hidden, size_t intermediate, size_t top_k, const float *input,
                    size_t input_len, float *output, size_t output_len, size_t n_tokens);

/* The sampler's candidate list on the device: the k largest of n fp32 values (logits or
 * probabilities), largest first, with their indices -- what the reference builds by sorting
 * (index, value) pairs and truncating to top_k (crates/oxillama-runtime/src/sampling/mod.rs:
 * 500-509); k = 1 is its argmax (mod.rs:652-662: the first of equal maxima).  Exactly equal values
 * come out lower index first (the reference's unstable sort leaves that open); NaNs rank last.
 * 1 <= k <= 256, k <= n <= 2^20.  Needs oxq_topk_workspace_bytes() bytes of 8-byte-aligned device
 * scratch; one or two launches (from k = 16 on vectors of more than 4096 values: slices of the
 * vector selected side by side, then their survivors by one work group), no allocation, no
 * synchronisation. */
size_t oxq_topk_workspace_bytes(size_t n, size_t k);
int oxq_topk_dev(const float *d_values, size_t n, size_t k, float *d_out_values,
                 uint32_t *d_out_indices, void *d_workspace, size_t workspace_bytes, void *stream);

/* The vocabulary projection and the candidate list of its logits in one call: d_logits[n_rows] = W . x as
 * oxq_matvec_q8_fused_dev computes it (accumulate = 0; the same bits), and the k largest logits with their row
 * indices as oxq_topk_dev lists them (same order, same ties) -- the lm_head's forward followed by the sampler's sort
 * and truncation (crates/oxillama-runtime/src/sampling/mod.rs:500-509; k = 1: its argmax, mod.rs:652-662) for a
 * request that edits no logits first (no banned tokens, bias or repetition penalty: those go through
 * oxq_logits_edit_dev between the two separate calls).  For k <= 8 (greedy decoding, small top_k) on Q6_K, Q8_0,
 * Q4_K, Q5_K, Q4_0 matrices whose rows take one wave (up to 8192 columns of the 256-weight formats, 4096 of the
 * others; at most 64 row batches per wave) this is ONE launch: every wave of the GEMV keeps its rows' logits as keys
 * and selects its k largest after its last row, the work group merges its waves' lists, and the last work group to
 * finish merges the work groups' lists (a ticket in library-owned device memory, which the launch leaves at zero;
 * no work group waits for another) -- 128256 x 4096 Q6_K with k = 1: 74.7 us against 78.2 for the separate launches.
 * Any other k, shape or format runs the GEMV launch and then oxq_topk_dev's launches, with the same results.
 * 1 <= k <= 256, k <= n_rows <= 2^20.  Needs oxq_lm_head_topk_workspace_bytes() bytes of 8-byte-aligned device
 * scratch.  No allocation, no synchronisation.  A HIP graph that holds such a launch must not run twice at the same
 * time (the ticket's address is part of the recorded launch). */
size_t oxq_lm_head_topk_workspace_bytes(uint32_t type, size_t n_rows, size_t n_cols, size_t k);
int oxq_lm_head_topk_dev(uint32_t type, const uint8_t *d_weights, const uint8_t *d_acts_q8, float *d_logits,
                         size_t n_rows, size_t n_cols, size_t k, float *d_out_values, uint32_t *d_out_indices,
                         void *d_workspace, size_t workspace_bytes, void *stream);

/* The sampler's edits of the logits BEFORE the candidate list, in place (sample_with_rng steps 0 and 1,
 * crates/oxillama-runtime/src/sampling/mod.rs:573-613): banned tokens to -inf; d_bias_values[i] added
 * to logit d_bias_tokens[i] where that logit is still finite (each token at most once: the
 * reference's map); the repetition penalty over the last `window` of the n_recent recent tokens --
 * once per occurrence, a positive logit divided by the penalty, any other multiplied; nothing for
 * a penalty of 1.  Token ids >= n are skipped, as in the reference.  Any list may be empty (NULL,
 * 0).  window <= 4096 entries in effect.  One launch; the grammar mask of the reference is not here. */
int oxq_logits_edit_dev(float *d_logits, size_t n, const uint32_t *d_banned, size_t n_banned,
                        const uint32_t *d_bias_tokens, const float *d_bias_values, size_t n_bias,
                        const uint32_t *d_recent, size_t n_recent, size_t window,
                        float repetition_penalty, void *stream);
/* The rest of the sampler on those candidates (sample_with_rng from its greedy shortcut on,
 * crates/oxillama-runtime/src/sampling/mod.rs:487-564): temperature <= 0 or k == 1 returns the
 * first candidate; otherwise every value times 1/temperature, softmax over the k candidates
 * (mod.rs:617-638), min-p (keep p >= min_p * p[0]; 0 = off), top-p (cut after the cumulative sum
 * reaches top_p; 1 = off), renormalisation, and the draw against one value of the reference's
 * Xorshift64 (mod.rs:669-690), whose state *d_rng_state holds and which advances only when more
 * than one candidate survives, as in the reference.  d_values / d_indices: k candidates, largest
 * value first (oxq_topk_dev's output; the values are the logits after whatever bias, penalty or
 * mask the caller applies -- those steps of the reference are not here).  *d_token receives the
 * token id; d_probs (optional, k floats) the final probabilities, zeros past the survivors.
 * 1 <= k <= 256.  Every fp32 operation is the reference's, in its order, so token and generator
 * state are the reference's for the same candidates (equal logits: see oxq_topk_dev).  One
 * launch, no allocation, no synchronisation.  Seed the state as Xorshift64::new does: the seed,
 * or 0x517cc1b727220a95 for a zero seed. */
int oxq_sample_candidates_dev(const float *d_values, const uint32_t *d_indices, size_t k,
                              float temperature, float min_p, float top_p, uint64_t *d_rng_state,
                              uint32_t *d_token, float *d_probs, void *stream);

int oxq_block_sums_dev(uint32_t type, const uint8_t *d_weights, const uint8_t *d_acts_q8,
                       int32_t *d_sums, size_t n_rows, size_t n_cols, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* OXQ_H */
