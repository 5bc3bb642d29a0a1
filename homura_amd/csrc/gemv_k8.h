// Q4_K / Q6_K decode product over the K8 form of the matrices (kquant_planes8.h). Internal.
#pragma once

#include "gemv_quant.h"
#include "hm_common.h"

namespace homura {

// out[n] = row n of the K8 matrix (plane [N][K], records [N][K / 8 + K / 64]) times the activation row d_x,
// which is prepared as `fuse` says (SiLU pair | residual add, RMSNorm) and quantised to Q8_K inside the launch;
// fuse.res_out_add is added on the way out. K % 256 == 0, K <= 16384 (8192 with a norm); no argmax candidates.
int gemv_k8_fused(hm_ctx *ctx, const float *d_x, const uint8_t *d_plane, const uint8_t *d_records, float *d_out, int K, int N,
                  const QuantFuse &fuse);

}  // namespace homura
