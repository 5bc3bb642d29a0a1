// Internal launch interface of the whole-step decode kernel (one launch for the embedding row
// and every decoder layer of a bf16 model), shared with the decode plan.
#pragma once
#include "hm_common.h"

// Weight formats the kernel has instances for.
// FUSED_WF_K8: Q4_K / Q6_K matrices (any mix) re-packed by kquant_planes8.hip: every weight as one signed byte,
// a scale and a minimum factor per 16 weights, the super-block's f16 d and dmin; multiplied as the reference
// multiplies K-quants, against the Q8_K quantisation of the activations in integer dot products.
enum : int { FUSED_WF_BF16 = 0, FUSED_WF_Q8_0 = 1, FUSED_WF_Q4_0 = 2, FUSED_WF_K8 = 3 };

// Per-layer device pointers. bf16: matrices in the K-contiguous stream layout the plan keeps:
// wqkv [q_dim + 2 kv_dim][hidden], wo [hidden][q_dim], wgu [2 inter][hidden] with gate and up rows
// interleaved (g0, u0, g1, u1, ...), wd [hidden][inter]; the s* pointers are unused. Q8_0 / Q4_0: w* are the
// quant planes and s* the scale planes of the same matrices re-packed as gemv_quant_planes.hip describes,
// q|k|v stacked in that order, wgu all gate rows and then all up rows. K8: w* the byte planes [N][K], s* the
// per-row scale records (kquant_planes8.h), same row order.
struct FusedLayerPtrs {
    const void *wqkv, *wo, *wgu, *wd;
    const uint16_t *sqkv, *so, *sgu, *sd;
    const float *in_ln, *post_ln;
    const float *q_norm, *k_norm;  // [head_dim] or nullptr (both)
    const float *qkv_bias;         // [q_dim + 2 kv_dim] or nullptr
    uint16_t *kcache, *vcache;     // [kv_heads][max_len][head_dim] bf16
};

struct FusedShape {
    int hidden, heads, kv_heads, head_dim, inter;
    int wf = FUSED_WF_BF16;  // FUSED_WF_*
};

struct FusedDecodeArgs {
    const FusedLayerPtrs *layers;  // device array [n_layers]
    int n_layers;
    const float *embed;  // [vocab][hidden] f32
    int vocab;
    const DecodeState *state;
    const int32_t *forced;
    float *hidden_out;  // [hidden]: the last layer's output (input of the LM head)
    const float *cos_tab, *sin_tab;  // [max_pos][head_dim]
    float eps, scale;
    int max_len;         // rows per KV head in the caches
    unsigned char *xch;  // exchange area, decode_fused_xch_bytes() bytes, zeroed once
    uint32_t *ctl;       // [0] launches so far (tag base), [1] sticky status (0 = ok), zeroed once
    // Optional LM head and greedy pick inside the same launch (head_w == nullptr: the launch ends with
    // hidden_out, as the layers' last output). head_w: bf16 [vocab][hidden] in the stream layout; head_norm: the
    // final RMSNorm weights; logits: [vocab] f32. With advance set, workgroup 0 finishes the step as
    // finish_step does: out_tokens[step] = pick (while step < out_cap), state->token = pick, step and pos + 1.
    const uint16_t *head_w;
    const float *head_norm;
    float *logits;
    DecodeState *state_rw;
    int32_t *out_tokens;
    int out_cap;
    int advance;
    // 1: take every exchange through memory, as a step does whose workgroups the placement check does not
    // find dealt to the dies round-robin (for tests of that path; the host sets it from HOMURA_WHOLE_STEP_FAR)
    int far_only;
    // Test support. spin_limit > 0: a wait gives up after that many polls instead of 2^20. withhold_wg >= 0: that
    // workgroup does not publish its Q|K|V rows of layer 0, so every wait for them runs into its bound, all
    // workgroups walk on without waiting, and the launch ends normally with the status word set.
    int spin_limit;
    int withhold_wg;
    // Optional phase trace (nullptr = off; room for FUSED_TRACE_WGS workgroups x (11 n_layers + 2) entries):
    // every workgroup stores, in its own row, the 100 MHz device clock at 11 points per
    // layer - both barriers of the Q|K|V, attention, O, gate|up and down phases, and the end of the fold
    // after attention's second barrier - followed by one entry at the end of the kernel and a last word that
    // is 1 when the step's exchanges went through the dies' L2s.
    unsigned long long *trace;
};
// ctl words: [0] launches so far, [1] first wait that gave up (0 = none), [2] steps that ran without die-local
// traffic, [3] warnings (FUSED_WARN_*)
enum : uint32_t {
    FUSED_WARN_TOKEN_RANGE = 1u,      // a fed-back token id lay outside the vocabulary and was replaced by 0
    FUSED_WARN_NO_FINITE_LOGIT = 2u,  // the greedy pick found no finite logit and took token 0
};
constexpr int FUSED_TRACE_PER_LAYER = 11;
constexpr int FUSED_TRACE_WGS = 256;  // rows of the trace buffer (the largest grid of any instance)

// Whether a kernel instance exists for this shape on this device (the cache may be of any length; a step is
// served while its live rows, the new one included, are at most decode_fused_max_kv). `why` receives a short
// reason when not.
bool decode_fused_supported(const hm_ctx *ctx, const FusedShape &s, int n_layers, int max_seq_len, const char **why);
size_t decode_fused_xch_bytes(const FusedShape &s);
// Most live cache rows (the new one included) the attention phase serves for this shape (0 if unsupported)
int decode_fused_max_kv(const FusedShape &s);
// The instances of a shape differ in how many live rows they hold (the ones that hold fewer are faster): the
// capacity of the instance that a step with `live_rows` live rows takes, 0 if none serves it. A recorded
// launch stays good while this value does not change.
int decode_fused_tier(const FusedShape &s, int live_rows);
// live_rows: the cache rows of the step, the new one included (the host's count; the kernel reads the position
// from the cursor and leaves with a status code if it does not fit the instance).
int decode_fused_launch(hm_ctx *ctx, const FusedShape &s, const FusedDecodeArgs &a, int live_rows);
// Reads the sticky status words (synchronises the stream). HM_OK, or HM_ERR_HIP with a message; *gave_up (when
// given) tells a wait that ran into its bound, which the caller can recover from, from the other failures.
int decode_fused_check(hm_ctx *ctx, const uint32_t *d_ctl, bool *gave_up = nullptr);
// The same verdict from a host copy of the 16 control words.
int decode_fused_check_words(hm_ctx *ctx, const uint32_t *h_ctl, bool *gave_up);
