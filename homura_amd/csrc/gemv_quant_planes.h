// Launch interface of the Q8_0 / Q4_0 GEMV over re-packed weights ("planes": all quant bytes row after
// row, then all f16 scales row after row; the same bytes as the GGUF blocks), shared with the model.
#pragma once

#include <cstddef>
#include <cstdint>

#include "gemv_quant.h"
#include "hm_common.h"

namespace homura {

// Bytes of the planes of an [N][K] matrix, and where the scale plane starts (256-byte aligned).
size_t quant_planes_bytes(bool q4, int N, int K);
size_t quant_planes_scale_offset(bool q4, int N, int K);

// raw blocks [N][K / 32] -> planes (one launch, at upload)
int pack_quant_planes(hm_ctx *ctx, bool q4, const uint8_t *d_blocks, uint8_t *d_planes, int N, int K);

// out[N] = W[N][K] . f(x) with the light ops of QuantFuse, W as planes; K <= 4096
int gemv_planes_fused(hm_ctx *ctx, bool q4, const float *d_x, const uint8_t *d_planes, float *d_out, int K, int N,
                      const QuantFuse &fuse);

// Workgroups gemv_planes_fused launches for this shape (= argmax candidates it leaves when asked to).
int gemv_planes_workgroups(const hm_ctx *ctx, bool q4, int K, int N);

// Q6_K [N][K] re-packed into four planes (nibbles, top bits, scales, block scales: the bytes of the blocks,
// every run at its natural alignment) and the f32 product over them: out[N] = dequant(W) . x, with the row's
// RMSNorm in front when d_norm_w is set and the workgroups' argmax candidates behind when cand_v is set.
// The product serves K = 256, 512, 1024, 2048 and 4096 (q6k_planes_shape_ok); packing any multiple of 256.
bool q6k_planes_shape_ok(int N, int K);
size_t q6k_planes_bytes(int N, int K);
int pack_q6k_planes(hm_ctx *ctx, const uint8_t *d_blocks, uint8_t *d_planes, int N, int K, bool unpack);
int dequant_q6k_planes(hm_ctx *ctx, const uint8_t *d_planes, float *d_out, int N, int K);
int gemv_q6k_planes_f32(hm_ctx *ctx, const char *name, const float *d_x, const float *d_norm_w, float eps, const uint8_t *d_planes,
                        float *d_out, int M, int K, int N, float *cand_v, int *cand_i, int cand_cap);
// Workgroups that product launches (= argmax candidates it leaves), capped at cand_cap when that is positive.
int q6k_planes_workgroups(const hm_ctx *ctx, int K, int N, int cand_cap);

}  // namespace homura
