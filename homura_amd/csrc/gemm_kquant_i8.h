// K-quant projections of a prompt chunk on the int8 matrix cores. Internal.
//
// The reference multiplies Q4_K / Q6_K blocks with Q8_K-quantised activation rows in integers
// (src/graph_builder/emit_quant.rs:165-816): per 256-wide block of a row
//     d * a * sum_sub sc_sub * (q . x)_sub  -  dmin * a * sum_sub mn_sub * sum(x)_sub
// with x the row's int8 values and a its scale. Both sums are dot products over k of x with small integers:
// sc_sub(k) * q_k (at most 13 bits) and mn_sub(k) (6 bits). A weight matrix is therefore re-packed once into
// three int8 "digit planes" [3][N][K]:
//     plane 0 (hi), plane 1 (lo):  sc * q = 128 * hi + lo,  lo in [-64, 63]
//     plane 2 (mn):                the minimum factor of k's sub-block (Q6_K: 0)
// and per (row, block) the two f32 scales (d, dmin). `v_mfma_i32_32x32x32_i8` adds up the three products over a
// block exactly; the block's value is then float(128 S_hi + S_lo) * (d a) - float(S_mn) * (dmin a), the
// arithmetic of the decode kernels (gemv_kquant.hip), blocks added in ascending order.
#pragma once

#include <cstdint>

#include "hm_common.h"

namespace homura {

inline size_t kq_i8_plane_bytes(int N, int K) { return 3 * (size_t)N * K; }
inline size_t kq_i8_scale_bytes(int N, int K) { return (size_t)N * (K / 256) * 2 * sizeof(float); }

// Re-packs `rows` rows of raw blocks (HM_DTYPE_Q4_K or HM_DTYPE_Q6_K, K % 256 == 0) into rows
// r * row_mult + row_off of the digit planes (N_total rows each) and of the scales [N_total][K / 256][2].
int kq_i8_pack(hm_ctx *ctx, int hm_dtype, const uint8_t *d_blocks, int rows, int K, int8_t *d_planes, float *d_scales,
               int N_total, int row_mult, int row_off);

// f32 rows -> Q8_K rows (reference quantize_row_q8_k: amax / 127, round half to even, clamp to +-127):
// d_q [rows][dim] int8, d_scale [rows][dim / 256] f32. dim % 256 == 0.
int quantize_q8k_rows_launch(hm_ctx *ctx, const float *d_x, int8_t *d_q, float *d_scale, size_t rows, int dim);

// C [M][N] f32 (row stride ldc, 0 = N) = Q8_K rows x K-quant matrix^T. With `parts`, K may be cut into up to
// max_parts slices of whole blocks written as [parts][M][ldc], to be added in index order by the consumer.
int gemm_q8k_kquant_nk(hm_ctx *ctx, const int8_t *d_aq, const float *d_ascale, const int8_t *d_planes,
                       const float *d_scales, float *d_c, int M, int K, int N, int max_parts = 1, int *parts = nullptr,
                       int ldc = 0);

}  // namespace homura
