// Internal launch interfaces of the light ops, shared with the decode plan.
#pragma once
#include "hm_common.h"

struct QkRopeArgs {
    float *q = nullptr;              // [S][H][hd], in place
    float *k = nullptr;              // [S][kvh][hd], in place
    const float *qw = nullptr;       // [hd] or NULL
    const float *kw = nullptr;       // [hd] or NULL
    const float *cos = nullptr;      // [S][hd]
    const float *sin = nullptr;      // [S][hd]
    int S = 0, H = 0, kvh = 0, hd = 0;
    float eps = 0.f;
    // optional fused cache append (batch 1): v [S][kvh][hd] f32, caches [kvh][max_len][hd] bf16
    const float *v = nullptr;
    uint16_t *kcache = nullptr;
    uint16_t *vcache = nullptr;
    int max_len = 0, pos = 0;
    // Decode-plan mode: the row position comes from state->pos and cos/sin point at the FULL
    // tables [max_pos][hd] (row pos + s is used), instead of pre-sliced rows.
    const DecodeState *state = nullptr;
};

int qknorm_rope_launch(hm_ctx *ctx, const QkRopeArgs &a);
// out = rmsnorm(x [+ res]) * w per row; resid_out (optional) receives x + res
int rmsnorm_launch(hm_ctx *ctx, const float *d_x, const float *d_res, const float *d_w, float *d_out,
                   float *d_resid_out, int rows, int dim, float eps);
int embed_launch(hm_ctx *ctx, const int64_t *d_ids64, const int32_t *d_ids32, const float *d_table,
                 float *d_out, int n_ids, int vocab, int hidden);
int argmax_candidates_launch(hm_ctx *ctx, const float *d_vals, const int *d_idxs, int n,
                             int32_t *d_out);
// Decode-plan variants driven by the device-resident cursor:
// embedding of this step's input id (forced id while step < n_forced, else the last pick)
int embed_step_launch(hm_ctx *ctx, const DecodeState *state, const int32_t *d_forced,
                      const float *d_table, float *d_out, int vocab, int hidden);
// fold the LM-head argmax candidates, record the pick, advance the cursor
int finish_step_launch(hm_ctx *ctx, DecodeState *state, const float *d_vals, const int *d_idxs,
                       int n, int32_t *d_out_tokens, int out_cap);
