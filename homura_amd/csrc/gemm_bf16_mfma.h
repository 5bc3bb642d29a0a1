// Internal launch interface of the MFMA GEMM used by the prefill path.
#pragma once

#include <cstdint>

#include "hm_common.h"

namespace homura {

// C[M][N] f32 = (sum of the pieces of A)[M][K] x B[N][K]^T. d_a_split is [M][pieces * K] bf16: piece p
// of every f32 activation in columns [p K, (p+1) K) (what the kernels of prefill.hip write). B is the
// K-contiguous stream layout of the model weights. K % 32 == 0, pieces 1..3.
// With parts != NULL the product may be cut along K into up to max_parts slices when M x N alone
// leaves most of the chip idle: slice s lands in d_c + s * M * N, *parts says how many there are, and
// the caller adds them up in index order (d_c must hold max_parts * M * N floats).
int gemm_split_nk(hm_ctx *ctx, const uint16_t *d_a_split, int pieces, const uint16_t *d_b_nk, float *d_c, int M, int K,
                  int N, int max_parts = 1, int *parts = nullptr);

// The same sum of piece products against B in the reference's layout [K][N] (N contiguous; N % 8 == 0, K % 32 == 0).
int gemm_split_kn(hm_ctx *ctx, const uint16_t *d_a_split, int pieces, const uint16_t *d_b_kn, float *d_c, int M, int K,
                  int N);

// C = A x B^T for two f32 matrices, each given as three bf16 pieces per element: d_a_split [M][3 K],
// d_b_split [N][3 K] (piece p in columns [p K, (p+1) K)). The six products of an A piece and a B piece
// whose indices add up to at most 2 are accumulated; what is left out is below 2^-24 of the result.
// K % 64 == 0. Row r of C starts at d_c + r * ldc (ldc = 0: N); slices as in gemm_split_nk, slice s at
// d_c + s * M * ldc.
int gemm_split_split_nk(hm_ctx *ctx, const uint16_t *d_a_split, const uint16_t *d_b_split, float *d_c, int M, int K,
                        int N, int max_parts = 1, int *parts = nullptr, int ldc = 0);

// The same products with every tile loaded once (gemm_pieces_mfma.hip): a_pieces x b_pieces = 2 x 1 or 3 x 1
// (d_b_split is then the plain [N][K] bf16 matrix) or 3 x 3. K % 32 == 0. Slices and ldc as above.
int gemm_pieces_nk(hm_ctx *ctx, const uint16_t *d_a_split, int a_pieces, const uint16_t *d_b_split, int b_pieces,
                   float *d_c, int M, int K, int N, int max_parts = 1, int *parts = nullptr, int ldc = 0);

// 3 x 1 pieces against a block-scaled integer matrix: d_b_ints [N][K] bf16 holds the integers of a Q8_0 / Q4_0
// matrix (exact), d_scales [K / 32][npad] f32 the scale of every 32-wide block of every row (npad >= N rounded
// up to 128). C = sum over blocks of scale * (A x ints^T over the block). Slices and ldc as above.
int gemm_pieces_scaled_nk(hm_ctx *ctx, const uint16_t *d_a_split, const uint16_t *d_b_ints, const float *d_scales, int npad,
                          float *d_c, int M, int K, int N, int max_parts = 1, int *parts = nullptr, int ldc = 0);
int gemm_pieces_any(hm_ctx *ctx, const uint16_t *d_a_split, int a_pieces, const uint16_t *d_b_split, int b_pieces,
                    const float *d_scales, int npad, float *d_c, int M, int K, int N, int max_parts, int *parts, int ldc);

}  // namespace homura
