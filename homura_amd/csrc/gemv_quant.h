// Launch interface of the Q8_0 / Q4_0 GEMV with the neighbouring light ops of the reference's
// quantised plan folded in (src/hf/emitter_quant.rs:713-791 RMSNorm, :985-1071 Residual+Norm,
// :1077-1103 SiLU*Up, :1109-1134 ResAdd): they run while the activation row is staged, or on the
// way out, instead of as launches of their own.
#pragma once

#include <cstdint>

#include "hm_common.h"

namespace homura {

struct QuantFuse {
    // activation on the way in:  x <- silu(x) * x2                (x2 set)
    //                            x <- x + res_in                   (res_in set; resid_out, if set, receives it)
    //                            x <- (x * rsqrt(mean(x^2) + eps)) * norm_w   (norm_w set; K <= 4096)
    const float *x2 = nullptr;
    const float *res_in = nullptr;
    float *resid_out = nullptr;
    const float *norm_w = nullptr;
    float eps = 0.f;
    // result on the way out:     out[n] <- dot[n] + res_out_add[n]
    const float *res_out_add = nullptr;
    // (K8 product only) rows come in (gate_i, up_i) pairs: out[i] <- silu(dot[2 i]) * dot[2 i + 1], N / 2 results
    bool silu_pairs = false;
    // LM head: the best (value, last index among equals; -1 without rows) of every workgroup, one entry
    // per workgroup of the launch (gemv_quant_workgroups of them)
    float *cand_v = nullptr;
    int *cand_i = nullptr;
};

// out[N] = W[N][K] (Q8_0 when q4 is false, Q4_0 when true) . f(x), one activation row
int gemv_quant_fused(hm_ctx *ctx, bool q4, const float *d_x, const uint8_t *d_w, float *d_out, int K, int N,
                     const QuantFuse &fuse);

// Workgroups gemv_quant_fused launches for this shape (= argmax candidates it leaves when asked to).
int gemv_quant_workgroups(const hm_ctx *ctx, bool q4, int K, int N);

}  // namespace homura
