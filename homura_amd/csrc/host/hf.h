// HF-style decoder model on the GPU plan: TransformerConfig, TransformerWeights, the plan
// emitters and HfModel (reference src/hf/config.rs, src/hf/weights.rs, src/hf/emitter.rs,
// src/hf/emitter_quant.rs, src/hf/model.rs).
#pragma once

#include <map>
#include <memory>
#include <string>
#include <vector>

#include "runtime.h"

namespace homura {

// reference TransformerConfig (src/hf/config.rs:11-73)
struct TransformerConfig {
    int hidden_size = 0, intermediate_size = 0, num_attention_heads = 0, num_hidden_layers = 0;
    int num_key_value_heads = 0;  // 0 => MHA
    int vocab_size = 0;
    double rms_norm_eps = 1e-6;
    double rope_theta = 10000.0;
    int max_position_embeddings = 2048;
    bool tie_word_embeddings = false;
    int head_dim_opt = 0;  // 0 => hidden_size / num_attention_heads
    bool attention_bias = false;  // q/k/v_proj.bias present (reference src/hf/weights.rs:64-69)
    int eos_token_id = -1, bos_token_id = -1;  // -1: none (reference Option<u32>)

    int kv_heads() const { return num_key_value_heads ? num_key_value_heads : num_attention_heads; }
    int head_dim() const { return head_dim_opt ? head_dim_opt : hidden_size / num_attention_heads; }
    int gqa_repeat() const { return num_attention_heads / kv_heads(); }
    int q_dim() const { return num_attention_heads * head_dim(); }
    int kv_dim() const { return kv_heads() * head_dim(); }
};

// One entry of TransformerWeights::to_slot_buffers (src/hf/weights.rs:63-116 / :136-183):
// what the host hands over for this slot.
struct WeightSlotInfo {
    std::string name;
    DType dtype;
    int64_t dim0 = 0, dim1 = 0;  // bf16/f32 matrices: [K][N] as the reference keeps them;
                                 // quantised: dim0 = N rows, dim1 = K (raw blocks [N][K/32])
    size_t bytes = 0;
};

// Scratch that the reference's fused kernels keep internal (attention output before the
// O projection, the MLP's residual and activation) plus the LM-head argmax candidates.
struct PlanScratch {
    Buffer attn_flat, resid, act, cand_val, cand_idx;
    // whole-step decode launch (bf16 plans of a served shape): device layer table, exchange area,
    // control words {launch count, status}
    Buffer fused_layers, fused_xch, fused_ctl, fused_trace;
    // test support (hm_model_whole_step_inject_timeout): handed to the next whole-step launches
    int inject_spin_limit = 0, inject_withhold_wg = -1;
    Buffer normed, gate, up, down, q_raw, k_raw, v_raw;  // quantised plan only
    int cand_cap = 0;
};

class HfModel {
  public:
    // proj_dtypes: optional, 7 per layer (q, k, v, o, gate, up, down) for a quantised model whose
    // projections do not all share weight_dtype.
    static std::unique_ptr<HfModel> create(hm_ctx *ctx, const TransformerConfig &cfg, DType weight_dtype,
                                           bool has_qk_norm, const std::vector<DType> *proj_dtypes = nullptr);
    DType proj_dtype(int layer, int which) const { return proj_dtypes_[(size_t)layer * 7 + which]; }
    ~HfModel();

    const TransformerConfig &config() const { return cfg_; }
    bool has_qk_norm() const { return has_qk_norm_; }
    DType weight_dtype() const { return weight_dtype_; }
    const std::vector<WeightSlotInfo> &weight_slot_infos() const { return infos_; }
    // Upload one slot (host pointer, exact byte size). bf16 matrices arrive [K][N] and are
    // re-packed once into the K-contiguous stream layout; quantised blocks stay as they are.
    int set_weight(int slot, const void *h_data, size_t bytes) { return set_weight_impl(slot, h_data, bytes, false); }
    // Same, but a matrix slot (bf16 projection, LM head) arrives [N][K] - one output row after the
    // other, K contiguous: the layout of HF safetensors ([out, in]) and of GGUF tensors, and the
    // stream layout kept in HBM, so nothing is transposed on the way in.
    int set_weight_nk(int slot, const void *h_data, size_t bytes) { return set_weight_impl(slot, h_data, bytes, true); }
    // Block-quantised plans only, before finalize: the LM head as the GGUF blocks of the output matrix
    // (Q8_0, Q4_0, Q4_K or Q6_K, rows of hidden / 32 or hidden / 256 blocks) in place of the f32 slot. The head
    // then multiplies the f32 row with the dequantised weights straight from the blocks - the numbers of the
    // reference's f32 head over the matrix its loader dequantises (src/gguf.rs:589-708, :696-700), read at a
    // sixth to a quarter of the bytes. hidden a multiple of the block length, at most 4096.
    int set_lm_head_blocks(DType dtype, const void *h_blocks, size_t bytes);
    // reference HfModel::ensure_compiled (src/hf/model.rs:148-160) + RoPE tables (:62-66)
    int finalize(int max_seq_len);

    // reference HfModel::run_kv (src/hf/model.rs:198-218); multi-token input is consumed one
    // token per plan step. h_logits: [n_ids][vocab] or NULL.
    int run_kv(const int64_t *h_ids, int n_ids, float *h_logits);
    // The multi-token pass behind run_kv for longer inputs (reference run_kv with seq > 1,
    // src/hf/model.rs:321-336): the chunk goes through the layers as a matrix, projections on the
    // matrix cores, causal attention over cache + chunk; n_ids rows are appended to the KV cache.
    // bf16 plan, head_dim 64 or 128. h_logits: [n_ids][vocab] or NULL (then the LM head is skipped).
    int prefill(const int64_t *h_ids, int n_ids, float *h_logits);
    bool prefill_available() const;
    // Inputs of at least this many tokens take the prefill pass (0 = never). Default 8.
    void set_prefill_min(int n) { prefill_min_ = n; }
    int prefill_min() const { return prefill_min_; }
    // bf16 pieces per f32 activation in the prefill pass: 3 (all 24 significant bits, default) or 2
    // (16 bits, two thirds of the matrix-core work)
    void set_prefill_pieces(int n) { prefill_pieces_ = n; }
    // Block-quantised models: HBM the prompt pass may keep for the dequantised projections (three bf16
    // pieces per weight, 6 bytes). When all of them fit, they are written once and stay; otherwise
    // (or with 0) every chunk dequantises them again into one scratch matrix.
    void set_prefill_weight_cache(size_t bytes);
    int init_kv_cache(const float *const *h_kv, int seq_len);
    int reset_kv_cache();
    int kv_cache_len() const;
    int generate_greedy(const int64_t *h_prompt, int n_prompt, int n_new, int32_t *h_tokens);
    // reference generate_streaming_core (src/generate.rs:100-315) with sample_token (:698-801)
    int generate(const int64_t *h_prompt, int n_prompt, int max_new, const hm_sampling_config &cfg, uint64_t seed,
                 int eos_token, int32_t *h_tokens, int *n_out);
    int bench_decode(int64_t first_id, int n_steps, float *ms_out, int32_t *h_tokens);
    int profile_step(int64_t token_id, std::vector<StepProfile> &out);
    // The whole-step decode launch (one kernel for the embedding row and all layers) instead of one
    // launch per projection. Available for bf16 models of a served shape; on by default then.
    bool whole_step_available() const { return fused_available_; }
    int set_whole_step(bool on);
    bool whole_step() const { return plan_ && plan_->whole_step(); }
    // HM_OK, or the error a whole-step launch left behind. A wait that ran into its bound is recovered from by
    // the call that met it (the steps of that call run again, one launch per projection, and so do later
    // calls); it stays reported here until reset_kv_cache or set_whole_step(true) re-arms the launch.
    int whole_step_status();
    // Test support: the next whole-step launches give up a wait after `spin_limit` polls, and workgroup
    // `workgroup` withholds its first publish, so that every workgroup runs into that bound and leaves normally.
    int whole_step_inject_timeout(int workgroup, int spin_limit);
    // Phase trace of the latest whole-step launch (device clock ticks at 100 MHz; 11 entries per layer
    // and a final one, see decode_fused.h). Recording starts with the first call, which returns 0
    // entries; later calls return the trace of the step that ran last.
    int whole_step_trace(unsigned long long *h_out, int cap, int *n_out);
    // Test support: keep the activation rows that the prompt pass hands to the Q8_K quantiser for the next
    // `rows` cache positions (0 = stop and free), and copy them out (layout at PrefillScratch::capture).
    int prefill_capture_q8k_inputs(int rows);
    int prefill_captured_q8k_inputs(float *h_out, size_t n_floats);
    int time_kernels(int rounds, std::vector<StepProfile> &out);
    ExecutionPlan *plan() { return plan_.get(); }

  private:
    HfModel() = default;
    int set_weight_impl(int slot, const void *h_data, size_t bytes, bool nk_layout);
    int emit_transformer_plan();        // reference src/hf/emitter.rs:867-1050
    int emit_transformer_plan_quant();  // reference src/hf/emitter_quant.rs:1142-1503
    int step_inputs(std::vector<Buffer *> &inputs);
    int refresh_fused_table();
    int finish_sync();
    int recover_whole_step();
    // the bodies of the calls of the same name, which run them again after a recovered whole-step timeout
    int run_kv_once(const int64_t *h_ids, int n_ids, float *h_logits);
    int generate_greedy_once(const int64_t *h_prompt, int n_prompt, int n_new, int32_t *h_tokens);
    int generate_once(const int64_t *h_prompt, int n_prompt, int max_new, const hm_sampling_config &cfg, uint64_t seed,
                      int eos_token, int32_t *h_tokens, int *n_out);
    int bench_decode_once(int64_t first_id, int n_steps, float *ms_out, int32_t *h_tokens);
    template <class Body>
    int with_whole_step_retry(Body body);
    int prefill_chunk(const int32_t *h_ids, int n, float *h_logits);
    const float *weight_f32(const std::string &name) const;
    int check_ids(const int64_t *ids, int n, std::vector<int32_t> &out);

    hm_ctx *ctx_ = nullptr;
    TransformerConfig cfg_;
    DType weight_dtype_ = DType::BF16;
    bool has_qk_norm_ = false;
    bool finalized_ = false;
    bool fused_available_ = false;
    int fused_max_kv_ = 0;            // live cache rows (the new one included) a whole-step launch serves
    int fused_tier_ = 0;              // capacity of the kernel instance the recorded step launches
    bool whole_step_wanted_ = false;  // the caller's choice; the plan follows it while the cache is short enough
    bool fused_dirty_ = false;        // whole-step launches were enqueued since the status words were last read
    bool fused_gave_up_ = false;      // a launch ran into a wait's bound: one launch per projection until re-armed
    std::string fused_gave_up_msg_;
    // pinned host staging of run_kv: a logits row and the whole-step status words arrive with one synchronisation
    void *h_stage_ = nullptr;
    size_t h_stage_bytes_ = 0;
    int check_fused_words(const uint32_t *h_ctl);
    int fused_wf_ = 0;  // FUSED_WF_* of the whole-step kernel instance
    bool fused_head_ = false;  // the whole-step launch also runs the LM head and the greedy pick (bf16 plan)
    const void *fused_table_kv_ = nullptr;  // key_ptr(0) the device layer table was built for
    int fused_table_max_len_ = 0;
    int max_seq_len_ = 0;
    std::vector<DType> proj_dtypes_;    // [layers][7]
    std::vector<WeightSlotInfo> infos_;
    std::vector<Buffer> weight_bufs_;   // in weight_slots order, device resident
    std::vector<bool> weight_set_;
    // packed storage the bf16 weight slot buffers are views of
    // qkv_bias: f32 [q_dim + 2 kv_dim]. quant[j] (j = q k v o gate up down) is set for the first
    // matrix of each run of same-type neighbours inside q|k|v and gate|up, and holds the whole run.
    // quant[first]: the raw blocks of a stacked run; planes[first]: the same run re-packed for the decode
    // GEMVs (Q8_0 / Q4_0 with K <= 4096; empty otherwise)
    // k8[g] (g = q|k|v, o, gate|up, down): a K-quant model's matrices re-packed for the whole-step launch
    // (kquant_planes8.h): the byte plane of the stacked rows, then their scale records
    struct LayerPacked { Buffer qkv, o, gate_up, down, qkv_bias, quant[7], planes[7], k8[4]; };
    int build_quant_planes();
    int build_k8_planes();
    // gate and up rows of the K8 form interleaved (g0, u0, g1, u1, ...): SiLU * up is then the epilogue of the
    // gate|up launch. Set for K-quant models that the whole-step launch does not serve (its instances read the
    // rows stacked).
    bool k8_pairs_ = false;
    // First member and member count of the stacked run that projection `which` of `layer` belongs to.
    void quant_run(int layer, int which, int *first, int *count) const;
    std::vector<LayerPacked> packed_;
    Buffer lm_head_packed_;
    Buffer lm_head_blocks_;             // set_lm_head_blocks: raw blocks of the output matrix
    Buffer lm_head_planes_;             // Q8_0 / Q4_0 output matrix re-packed for the decode GEMV
    DType lm_head_blocks_dtype_ = DType::F32;
    Buffer rope_cos_, rope_sin_;        // [max_position][head_dim] f32
    Buffer ids_view_, mask_view_;
    std::shared_ptr<PlanScratch> scratch_;
    // prefill pass: activations of one chunk of rows
    struct PrefillScratch {
        static constexpr int MAX_PARTS = 8;  // K slices a projection result may come in
        int rows = 0;
        Buffer ids, h, resid, split, qkv, proj_out, gate_up, logits;
        Buffer wsplit;  // block formats: the matrices of one group of projections as three bf16 pieces per weight
        std::vector<Buffer> wcache;  // [layer * 4 + group] resident copies of the same (q|k|v, o, gate|up, down)
        // K-quant groups on the integer matrix cores: the chunk's Q8_K rows (int8 values, one f32 scale per
        // 256) and, per [layer * 4 + group], the group's int8 digit planes followed by its block scales
        Buffer q8, q8s;
        std::vector<Buffer> icache;
        bool icache_off = false;  // the planes did not fit: K-quant groups keep the bf16 pieces
        // Q8_0 / Q4_0 groups: per [layer * 4 + group] the group's integers as bf16 followed by its block
        // scales [K / 32][N rounded up to 128] (gemm_pieces_scaled_nk)
        std::vector<Buffer> scache;
        bool scache_off = false;
        // Tests: the f32 rows entering the Q8_K quantisation of the K-quant products, for cache positions
        // [capture_base, capture_base + capture_rows); per layer [rows][hidden] (q|k|v), [rows][q_dim] (o),
        // [rows][hidden] (gate|up), [rows][inter] (down).
        Buffer capture;
        int capture_rows = 0, capture_base = 0;
    };
    PrefillScratch pf_;
    struct SamplerScratch { Buffer work, counts, token, list, draws; int list_cap = 0, draws_cap = 0; } sampler_;
    int prefill_min_ = 8;
    int prefill_pieces_ = 3;
    size_t prefill_weight_cache_bytes_ = (size_t)32 << 30;
    std::map<std::string, int> slot_by_name_;
    std::unique_ptr<ExecutionPlan> plan_;
};

}  // namespace homura
