// K-quant GEMV launch used by the model plan (the public entry points hm_gemv_q4_k / hm_gemv_q6_k
// always quantise the activation first).
#pragma once

#include <cstdint>

#include "gemv_quant.h"
#include "hm_common.h"

namespace homura {

// Fused form for the model plan: the light ops in front of the product (QuantFuse: SiLU pair, residual
// add, RMSNorm) and the Q8_K quantisation of the resulting row all happen inside the GEMV kernel - every
// workgroup redoes them for the one row, which is cheaper than the launches they replace - and the
// residual add behind it rides on the way out. K <= 4096.
int gemv_kquant_fused(hm_ctx *ctx, bool q6, const float *d_x, const uint8_t *d_w, float *d_out, int K, int N,
                      const QuantFuse &fuse);

// The fused form over two matrices of the two different K-quant types that share the row (q|k in Q4_K with v in
// Q6_K, as Q4_K_M files have them): one launch, the row prepared once per workgroup. Residual and norm
// prologue only. K <= 4096.
int gemv_kquant_fused_pair(hm_ctx *ctx, bool first_q6, const float *d_x, const uint8_t *d_w, float *d_out, int N,
                           const uint8_t *d_w2, float *d_out2, int N2, int K, const QuantFuse &fuse);

// out[N] = W[N][K] (Q4_K when q6 is false, Q6_K when true) · x[K], x quantised to Q8_K first.
// reuse_activation: skip the quantisation and multiply against what the previous call on this
// context's stream left at the top of the workspace (same x, same K). Q4_K and Q6_K share the
// activation format, so a Q6_K matrix may follow a Q4_K one on the same x.
int gemv_kquant(hm_ctx *ctx, bool q6, const float *d_x, const uint8_t *d_w, float *d_out, int K, int N,
                bool reuse_activation);

// LM head over K-quant blocks with f32 activations (the product with the dequantised weights): RMSNorm of
// the row with norm_w on the way in, logits out, and the best (value, last index among equals; -1 without rows) of every workgroup in
// cand_v / cand_i; gemv_kquant_f32_head_candidates says how many candidates that launch leaves.
// K % 256 == 0, K <= 4096.
int gemv_kquant_f32_head(hm_ctx *ctx, bool q6, const float *d_x, const float *d_norm_w, float eps, const uint8_t *d_w,
                         float *d_out, int K, int N, float *cand_v, int *cand_i, int cand_cap);
int gemv_kquant_f32_head_candidates(const hm_ctx *ctx, bool q6, int K, int N, int cand_cap);

}  // namespace homura
