/* Internal to the CPU oracle (TEST INFRASTRUCTURE): the formats restated in oxq_oracle_more.c,
 * reached through the dispatchers of oxq_oracle.c. */
#ifndef OXQ_ORACLE_MORE_H
#define OXQ_ORACLE_MORE_H
#include <stddef.h>
#include <stdint.h>

int oxq_more_known(uint32_t type);
size_t oxq_more_block_size(uint32_t type);
size_t oxq_more_block_bytes(uint32_t type);
size_t oxq_more_groups_per_block(uint32_t type); /* integer groups: 32 weights, 16 for Q2_K / Q3_K */
void oxq_more_dequant(uint32_t type, const uint8_t *block, float *out);
float oxq_more_gemv_row(uint32_t type, const uint8_t *row, size_t bpr, size_t n_cols, const float *x);
float oxq_more_fused_row(uint32_t type, const uint8_t *row, size_t bpr, size_t n_cols, const uint8_t *acts);
void oxq_more_block_sums_row(uint32_t type, const uint8_t *row, size_t bpr, const uint8_t *acts, int32_t *sums);
float oxq_more_intdot_row(uint32_t type, const uint8_t *row, size_t bpr, const uint8_t *acts, int32_t *scratch);
#endif
