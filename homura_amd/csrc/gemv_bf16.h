// Internal launch interface of the [N][K] bf16 GEMV with fused prologue/epilogue, shared
// with the decode plan.
#pragma once
#include "hm_common.h"

enum GemvEpilogue {
    GEMV_EPI_NONE = 0,
    GEMV_EPI_RESIDUAL = 1,        // out = epilogue_residual + W.x   (reference src/hf/emitter.rs:804)
    GEMV_EPI_SILU_MUL_PAIRS = 2,  // rows (2i, 2i+1) = (gate_i, up_i); out[i] = silu(gate)*up
    GEMV_EPI_ARGMAX = 3,          // also emit one (max, last index) candidate per workgroup
};

struct GemvArgs {
    const float *x = nullptr;                  // [M][K]
    const void *w = nullptr;                   // [N][K] bf16 (or f32 when w_f32)
    bool w_f32 = false;
    float *out = nullptr;                      // [M][N] (or [M][N/2] for the paired epilogue)
    int K = 0, N = 0;
    // prologue: r = x + prologue_residual (optional), then RMSNorm with norm_w (optional)
    const float *prologue_residual = nullptr;  // [M][K]
    const float *norm_w = nullptr;             // [K]
    float eps = 0.f;
    float *resid_out = nullptr;                // [M][K]: receives r (written by one workgroup)
    const float *bias = nullptr;               // [N]: out = W.x + bias (reference src/hf/emitter.rs:604-619);
                                               // not with the paired epilogue
    const float *epilogue_residual = nullptr;  // [M][N]
    float *argmax_val = nullptr;               // [argmax_cap]
    int *argmax_idx = nullptr;                 // [argmax_cap]
    int argmax_cap = 0;
};

// Number of workgroups the launch will use for N output rows at R rows per wavefront.
int gemv_bf16_nk_grid(const hm_ctx *ctx, int N, int R);
// Enqueue on the context stream. For GEMV_EPI_ARGMAX the number of candidates written is
// min(gemv_bf16_nk_grid(ctx, N, 4), argmax_cap).
int gemv_bf16_nk_launch(hm_ctx *ctx, GemvArgs a, int M, int epi);
// [K][N] -> rows of an [.][K] stream-layout buffer: source column n becomes destination row
// n * row_mult + row_off.
int pack_bf16_kn_to_nk_strided(hm_ctx *ctx, const uint16_t *d_w_kn, uint16_t *d_dst, int K, int N,
                               int row_mult, int row_off);
int pack_f32_kn_to_nk(hm_ctx *ctx, const float *d_w_kn, float *d_dst, int K, int N);
