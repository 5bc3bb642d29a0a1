// Internal launch interface of the GQA decode attention kernel, shared with the decode plan.
#pragma once
#include "hm_common.h"

struct AttnArgs {
    const float *q = nullptr;          // [B][H][hd]
    const uint16_t *kcache = nullptr;  // [B][kvh][max_len][hd] bf16
    const uint16_t *vcache = nullptr;
    float *out = nullptr;              // [B][H*hd]
    int B = 0, H = 0, kvh = 0, hd = 0, max_len = 0, kv_len = 0;
    float scale = 1.f;
    // Decode-plan mode: kv_len = state->pos + 1 is read on the device and the grid is sized
    // for max_len with a fixed chunk (workgroups past the live range exit at once).
    const DecodeState *state = nullptr;
    int fixed_chunk = 0;
    // Decode-plan mode: rows the grid covers instead of max_len (0: max_len). The caller keeps
    // state->pos + 1 within it: rows beyond would not be looked at.
    int span = 0;
    // Fused prologue (decode plan, B == 1): when qkv_raw is set, q is ignored; the kernel applies
    // QK-norm + RoPE to the raw projection row and appends the new K/V row to the caches.
    const float *qkv_raw = nullptr;  // [H*hd | kvh*hd | kvh*hd]
    const float *qw = nullptr, *kw = nullptr;
    const float *cos_tab = nullptr, *sin_tab = nullptr;  // [max_pos][hd]
    float eps = 0.f;
    // which of the two kernels to enqueue: both (default), only the split attention, or only
    // the fold of its partials (the decode plan lists them as separate device launches)
    enum Phase { BOTH = 0, SPLIT_ONLY = 1, FOLD_ONLY = 2 };
    int phase = BOTH;
    // Where the splits' partial (o, max, sum) go: the context's workspace when null.
    float *partials = nullptr;
    size_t partials_bytes = 0;
};

// Resolves the device address of the library's fixed partials array on the context's device
// (called once per context by hm_init, with that device current).
int gqa_attn_fixed_scratch_setup(hm_ctx *ctx);

int gqa_decode_attn_launch(hm_ctx *ctx, const AttnArgs &a);
