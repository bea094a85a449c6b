/*
 * oxq_tuning.h -- launch-shape knobs of liboxq_hip.so for benchmarks and tests.
 *
 * Not part of the drop-in boundary: nothing here has a counterpart in the reference,
 * and the reference-side shim binds none of it.  Every knob is process-global, is
 * stored atomically and is read once per launch, so flipping one while other threads
 * are launching is safe; it changes which launch shape later calls take, never their
 * results (all shapes give the same integer sums; fp32 results differ only where the
 * summation order over a row differs, within the documented tolerance).  A value of 0
 * restores the built-in choice.
 */
#ifndef OXQ_TUNING_H
#define OXQ_TUNING_H

#ifdef __cplusplus
extern "C" {
#endif

/* Launch width of the GEMV kernels: resident waves per compute unit (tuning
 * knob for benchmarks; 0 restores the default). */
int oxq_set_gemv_waves_per_cu(unsigned waves);
/* Rows a wave loads per batch in the GEMV kernels (1, 2 or 4; tuning knob; 0 restores
 * the per-shape default). */
int oxq_set_gemv_rows_per_batch(unsigned rows);
/* Waves that share one row in the GEMV kernels (1 or 4; tuning knob; 0 restores the
 * per-shape default: 4 for rows of three or more 64-unit steps). */
int oxq_set_gemv_waves_per_row(unsigned waves);
/* Fewest activation rows for which oxq_gemm_q8_dev / oxq_gemm take the tile kernel; below it
 * they run GEMV launches, two to four rows per launch (tuning knob; 0 restores the default). */
int oxq_set_gemm_tile_min_rows(unsigned rows);
/* Which kernel and launch shape the batched matmuls take (tuning knob; 0 restores the default, the measured choice
 * per shape).  1..23: a fixed tile shape / prefetch depth of the int8-MFMA tile kernel; 99: the tile kernel's own
 * choice, never the few-token kernel nor the prefill kernel; 300: the prefill kernel (f16 matrix cores, Q4_K) for any
 * number of token rows; 200..205: the
 * few-token kernel (16 x 16 x 32 MFMA, groups of at most 32 token rows) in a fixed shape.  A value a format or
 * shape cannot take falls back to the default tile choice. */
int oxq_set_gemm_variant(int variant);
/* Launch-phase probe of the decode GEMV (Q4_0, Q8_0, Q4_K, Q6_K rows of at most two 64-unit steps, and the
 * fused gate + up launch): while d_buffer is set, those launches run an instantiation of the same kernel in
 * which every wave writes four uint64 words to d_buffer[(block * 4 + wave) * 4 ...]: three 100 MHz wall-clock
 * timestamps -- kernel entry, its first row batch stored, its last -- and where it ran (XCC_ID register in the
 * high half, HW_ID register in the low half).  Blocks of a multi-matrix launch are numbered matrix-major.  A launch that would not fit `bytes` runs unprobed.  NULL switches the probe off. */
int oxq_set_gemv_phase_probe(void *d_buffer, size_t bytes);
/* Which kernel instantiation and launch shape the calling thread's last GEMV / fused gate+up / tile-kernel
 * launch used, as "name<type,p0,p1,p2,p3> grid XxY block B" (template parameters in the kernel's own order):
 * lets a measurement name what it timed and notice when a launch policy has changed under it. */
int oxq_last_launch(char *out, size_t out_len);
/* oxq_ffn_swiglu_dev: 1 (default) = gate, up, SwiGLU and the quantizer of h in one launch where a kernel
 * exists for the type and row length; 0 = the separate launches (same bits). */
int oxq_set_ffn_fusion(int enabled);


#ifdef __cplusplus
}
#endif
#endif /* OXQ_TUNING_H */
