// Internal launch interfaces of the multi-token (prefill) kernels: a prompt chunk goes through
// the layers as a matrix, the projections run on the matrix cores.
//
// The reference multiplies f32 activations by bf16 weights (make_mixed_matmul_region,
// src/graph_builder/emit_linalg.rs:2224-2307). The MFMA takes bf16 on both sides, so every f32
// activation x is carried as bf16 pieces, p0 = bf16(x), p1 = bf16(x - p0), p2 = bf16(x - p0 - p1);
// the products of the pieces are summed in the f32 accumulator. Two pieces keep 16 significant bits
// of x, three keep all 24, which is what the path uses by default: K and V rows are rounded to bf16
// when they enter the cache, and activations that are off in the 17th bit flip that rounding for
// a few elements per row.
// A "split" matrix is [rows][pieces * dim] bf16: piece p in columns [p * dim, (p + 1) * dim).
#pragma once

#include <cstdint>

#include "hm_common.h"

namespace homura {

// A projection result may arrive as `parts` K slices of the GEMM, [parts][rows][dim] f32, to be added
// in index order (gemm_split_nk); the kernels below take the count next to the pointer.

// out_split = split(rmsnorm(x [+ res]) * w) per row; resid_out (optional, [rows][dim]) receives x + res.
// x: [rows][dim] f32; res: [res_parts][rows][dim] or NULL.
// q8k: the values go through the Q8_K quantisation of a K-quant product's activation first (per
// 256-wide block of the row, dim % 256 == 0), so the split matrix holds scale * q.
// d_pre_q8k (optional, [rows][dim] f32; tests): receives the values as they enter that quantisation.
// d_q8 / d_q8_scale (optional, with q8k): the Q8_K rows themselves, [rows][dim] int8 and [rows][dim / 256] f32,
// for the integer matrix cores (gemm_kquant_i8.h); no split matrix is written then.
int rmsnorm_split_launch(hm_ctx *ctx, const float *d_x, const float *d_res, int res_parts, const float *d_w,
                         uint16_t *d_out_split, int pieces, float *d_resid_out, int rows, int dim, float eps,
                         bool q8k = false, float *d_pre_q8k = nullptr, int8_t *d_q8 = nullptr, float *d_q8_scale = nullptr);

// out_split = split(x) (through Q8_K first with q8k); x: [rows][dim] f32, dim % 4 == 0
int split_rows_launch(hm_ctx *ctx, const float *d_x, uint16_t *d_out_split, int pieces, size_t rows, int dim,
                      bool q8k = false);

// A block-quantised matrix (raw GGUF blocks [N][K / block], hm_dtype one of HM_DTYPE_Q8_0 / Q4_0 / Q4_K /
// Q6_K) as the split matrix [.][3 K] of its dequantised f32 values (the bits of the reference's
// dequantisation, src/gguf.rs:825-917): row n lands in row n * row_mult + row_off.
int dequant_split_launch(hm_ctx *ctx, int hm_dtype, const uint8_t *d_blocks, int N, int K, uint16_t *d_out_split,
                         int row_mult = 1, int row_off = 0);


// A Q8_0 / Q4_0 matrix (raw GGUF blocks [N][K / 32]) as the operands of gemm_pieces_scaled_nk: its integers as
// bf16 (exact), row n in row n * row_mult + row_off of d_ints ([.][K]), and its block scales, d_scales
// [K / 32][npad] f32 (column = output row).
int quant_ints_launch(hm_ctx *ctx, int hm_dtype, const uint8_t *d_blocks, int N, int K, uint16_t *d_ints, float *d_scales,
                      int npad, int row_mult = 1, int row_off = 0);

// out_split = split(silu(gate) * up) for gate/up interleaved per row: gu [rows][2 * inter] =
// (gate_0, up_0, gate_1, up_1, ...), the column order of the packed gate|up weight.
int silu_mul_split_launch(hm_ctx *ctx, const float *d_gu, int parts, uint16_t *d_out_split, int pieces, int rows,
                          int inter, bool q8k = false, float *d_pre_q8k = nullptr, int8_t *d_q8 = nullptr,
                          float *d_q8_scale = nullptr);

// The tail of the reference's QKV kernel for S rows at positions past .. past + S - 1
// (src/hf/emitter.rs:604-649): bias add, per-head QK-norm, RoPE on q and k in place, and the
// append of the bf16-rounded k and v rows to the cache (KvCache::append_key / append_value,
// src/runtime.rs:521-568). qkv: [S][q_dim + 2 kv_dim] f32 rows (q | k | v).
struct QkvPostArgs {
    float *qkv = nullptr;                 // q is rewritten in place (slice 0)
    int parts = 1;                        // K slices of the projection
    size_t part_stride = 0;               // floats between slices
    const float *bias = nullptr;          // [q_dim + 2 kv_dim] or NULL
    const float *qw = nullptr, *kw = nullptr;  // [hd] or NULL
    const float *cos_tab = nullptr, *sin_tab = nullptr;  // full tables [max_pos][hd]
    uint16_t *kcache = nullptr, *vcache = nullptr;        // [kvh][max_len][hd] bf16
    int S = 0, H = 0, kvh = 0, hd = 0, max_len = 0, past = 0;
    float eps = 0.f;
};
int qkv_post_launch(hm_ctx *ctx, const QkvPostArgs &a);

// Causal GQA attention of S query rows (positions past .. past + S - 1) over cache rows
// [0, past + S): the attention part of the reference's attention kernel with the causal mask of
// build_causal_mask (src/hf/emitter.rs:709-737, src/hf/precompute.rs:134-161).
// q: f32 rows with stride ldq, head h at columns [h * hd, (h + 1) * hd). Output [S][H * hd] as f32
// (out_f32) and/or as a split matrix [S][pieces * H * hd] (out_split). hd = 64 or 128. q and the
// probabilities enter the MFMA as `pieces` (2 or 3) bf16 numbers each.
struct PrefillAttnArgs {
    const float *q = nullptr;
    int ldq = 0;
    const uint16_t *kcache = nullptr, *vcache = nullptr;  // [kvh][max_len][hd] bf16
    float *out_f32 = nullptr;
    uint16_t *out_split = nullptr;
    int S = 0, H = 0, kvh = 0, hd = 0, max_len = 0, past = 0;
    float scale = 1.f;
    int pieces = 3;
    // set by prefill_attn_launch when few query rows face a long cache: the keys are cut over gridDim.z
    // workgroups, which leave their (O, max, sum) here for a second kernel to join
    float *part_o = nullptr, *part_ml = nullptr;
};
int prefill_attn_launch(hm_ctx *ctx, const PrefillAttnArgs &a);

}  // namespace homura
