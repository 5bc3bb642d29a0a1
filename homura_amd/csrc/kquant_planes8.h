// Q4_K / Q6_K matrices re-packed for the whole-step decode kernel (its FUSED_WF_K8 format). Internal.
//
// The GGUF super-blocks (src/gguf.rs:835-917) keep a weight's bits in up to three places and their 6-bit
// scales packed; here every weight is one signed byte (Q4_K: the nibble 0..15; Q6_K: the 6-bit value - 32), in a
// plane [N][K], and every row has a scale record of K / 8 + K / 64 bytes: for each 16 weights the bytes (sc, mn)
// - the sub-block's scale and minimum factor (Q4_K: those of its 32-wide sub-block; Q6_K: its own int8 scale
// and 0) - then for each 256 weights the f16 bits (d, dmin) of the super-block (Q6_K: dmin = 0). With these the
// reference's K-quant product (src/graph_builder/emit_quant.rs:165-816) is the same integer arithmetic for
// both types: sum sc * isum and sum mn * bsum per super-block.
#pragma once
#include "hm_common.h"

inline size_t k8_plane_bytes(int N, int K) { return (size_t)N * K; }
inline size_t k8_record_bytes(int N, int K) { return (size_t)N * (K / 8 + K / 64); }
// Re-packs `rows` rows of raw blocks (hm_dtype HM_DTYPE_Q4_K or HM_DTYPE_Q6_K, K % 256 == 0) into rows
// row0, row0 + row_mult, row0 + 2 row_mult, ... of the byte plane d_plane and of the records d_records.
int pack_k8_rows(hm_ctx *ctx, int hm_dtype, const uint8_t *d_blocks, int rows, int K, uint8_t *d_plane, uint8_t *d_records,
                 int row0, int row_mult = 1);
