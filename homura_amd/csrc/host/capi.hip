// C handles onto the host classes (declared in include/homura_amd.h).
#include <cstring>

#include "hf.h"

using namespace homura;

struct hm_model {
    hm_ctx *ctx;
    std::unique_ptr<HfModel> impl;
};

extern "C" {

hm_model *hm_model_create(hm_ctx *ctx, const hm_transformer_config *cfg, int weight_dtype,
                          int has_qk_norm) {
    if (!ctx) return nullptr;
    if (!cfg) {
        hm_set_error(ctx, HM_ERR_INVALID, "hm_model_create: NULL config");
        return nullptr;
    }
    TransformerConfig c;
    c.hidden_size = cfg->hidden_size;
    c.intermediate_size = cfg->intermediate_size;
    c.num_attention_heads = cfg->num_attention_heads;
    c.num_hidden_layers = cfg->num_hidden_layers;
    c.num_key_value_heads = cfg->num_key_value_heads;
    c.vocab_size = cfg->vocab_size;
    c.head_dim_opt = cfg->head_dim;
    // reference defaults (src/hf/config.rs:39-47)
    c.max_position_embeddings = cfg->max_position_embeddings > 0 ? cfg->max_position_embeddings : 2048;
    c.tie_word_embeddings = cfg->tie_word_embeddings != 0;
    c.rms_norm_eps = cfg->rms_norm_eps > 0 ? cfg->rms_norm_eps : 1e-6;
    c.rope_theta = cfg->rope_theta > 0 ? cfg->rope_theta : 10000.0;
    c.attention_bias = cfg->attention_bias != 0;
    auto impl = HfModel::create(ctx, c, (DType)weight_dtype, has_qk_norm != 0);
    if (!impl) return nullptr;
    return new hm_model{ctx, std::move(impl)};
}

void hm_model_destroy(hm_model *m) { delete m; }

int hm_model_num_weight_slots(hm_model *m) {
    if (!m) return HM_ERR_INVALID;
    return (int)m->impl->weight_slot_infos().size();
}

int hm_model_weight_slot_info(hm_model *m, int slot, char *name_buf, size_t buflen, int *dtype,
                              int64_t *dim0, int64_t *dim1, size_t *bytes) {
    if (!m) return HM_ERR_INVALID;
    const auto &infos = m->impl->weight_slot_infos();
    if (slot < 0 || slot >= (int)infos.size())
        return hm_set_error(m->ctx, HM_ERR_INVALID, "weight slot %d out of range", slot);
    const WeightSlotInfo &w = infos[slot];
    if (name_buf && buflen) snprintf(name_buf, buflen, "%s", w.name.c_str());
    if (dtype) *dtype = (int)w.dtype;
    if (dim0) *dim0 = w.dim0;
    if (dim1) *dim1 = w.dim1;
    if (bytes) *bytes = w.bytes;
    return HM_OK;
}

int hm_model_set_weight(hm_model *m, int slot, const void *h_data, size_t bytes) {
    if (!m) return HM_ERR_INVALID;
    return m->impl->set_weight(slot, h_data, bytes);
}

int hm_model_finalize(hm_model *m, int max_seq_len) {
    if (!m) return HM_ERR_INVALID;
    return m->impl->finalize(max_seq_len);
}

int hm_model_init_kv_cache(hm_model *m, const float *const *h_kv, int seq_len) {
    if (!m) return HM_ERR_INVALID;
    if (!h_kv || seq_len < 0) return hm_set_error(m->ctx, HM_ERR_INVALID, "hm_model_init_kv_cache: bad arguments");
    return m->impl->init_kv_cache(h_kv, seq_len);
}

int hm_model_reset_kv_cache(hm_model *m) {
    if (!m) return HM_ERR_INVALID;
    return m->impl->reset_kv_cache();
}

int hm_model_kv_cache_len(hm_model *m) {
    if (!m) return HM_ERR_INVALID;
    return m->impl->kv_cache_len();
}

int hm_model_set_graph(hm_model *m, int on) {
    if (!m) return HM_ERR_INVALID;
    if (!m->impl->plan()) return hm_set_error(m->ctx, HM_ERR_STATE, "model not finalized");
    return m->impl->plan()->enable_graph(on != 0);
}

int hm_model_run_kv(hm_model *m, const int64_t *h_ids, int n_ids, float *h_logits) {
    if (!m) return HM_ERR_INVALID;
    return m->impl->run_kv(h_ids, n_ids, h_logits);
}

int hm_model_generate_greedy(hm_model *m, const int64_t *h_prompt, int n_prompt, int n_new,
                             int32_t *h_tokens_out) {
    if (!m) return HM_ERR_INVALID;
    return m->impl->generate_greedy(h_prompt, n_prompt, n_new, h_tokens_out);
}

int hm_model_bench_decode(hm_model *m, int64_t first_id, int n_steps, float *ms_out,
                          int32_t *h_tokens_out) {
    if (!m) return HM_ERR_INVALID;
    if (!ms_out) return hm_set_error(m->ctx, HM_ERR_INVALID, "hm_model_bench_decode: ms_out is NULL");
    return m->impl->bench_decode(first_id, n_steps, ms_out, h_tokens_out);
}

static int fill_profiles(const std::vector<StepProfile> &prof, hm_kernel_profile *out, int cap);

int hm_model_time_kernels(hm_model *m, int rounds, hm_kernel_profile *out, int cap) {
    if (!m) return HM_ERR_INVALID;
    std::vector<StepProfile> prof;
    int rc = m->impl->time_kernels(rounds, prof);
    if (rc != HM_OK) return rc;
    return fill_profiles(prof, out, cap);
}

int hm_model_launches_per_step(hm_model *m) {
    if (!m) return HM_ERR_INVALID;
    if (!m->impl->plan()) return hm_set_error(m->ctx, HM_ERR_STATE, "model not finalized");
    return m->impl->plan()->launches_per_step();
}

int hm_model_profile_step(hm_model *m, int64_t token_id, hm_kernel_profile *out, int cap) {
    if (!m) return HM_ERR_INVALID;
    std::vector<StepProfile> prof;
    int rc = m->impl->profile_step(token_id, prof);
    if (rc != HM_OK) return rc;
    return fill_profiles(prof, out, cap);
}

}  // extern "C"

static int fill_profiles(const std::vector<StepProfile> &prof, hm_kernel_profile *out, int cap) {
    int n = 0;
    for (auto &p : prof) {
        if (n >= cap) break;
        std::memset(&out[n], 0, sizeof(out[n]));
        snprintf(out[n].label, sizeof(out[n].label), "%s", p.label.c_str());
        out[n].ms = p.ms;
        out[n].launches = p.launches;
        out[n].bytes = p.bytes;
        n++;
    }
    return n;
}
