// K-quant GEMV launch used by the model plan (the public entry points hm_gemv_q4_k / hm_gemv_q6_k
// always quantise the activation first).
#pragma once

#include <cstdint>

#include "hm_common.h"

namespace homura {

// out[N] = W[N][K] (Q4_K when q6 is false, Q6_K when true) · x[K], x quantised to Q8_K first.
// reuse_activation: skip the quantisation and multiply against what the previous call on this
// context's stream left at the top of the workspace (same x, same K). Q4_K and Q6_K share the
// activation format, so a Q6_K matrix may follow a Q4_K one on the same x.
int gemv_kquant(hm_ctx *ctx, bool q6, const float *d_x, const uint8_t *d_w, float *d_out, int K, int N,
                bool reuse_activation);

}  // namespace homura
