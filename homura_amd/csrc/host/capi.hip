// C handles onto the host classes (declared in include/homura_amd.h).
#include <cstring>

#include "hf.h"
#include "../../../include/homura_amd_bench.h"
#include "loaders.h"

using namespace homura;

struct hm_model {
    hm_ctx *ctx;
    std::unique_ptr<HfModel> impl;
};

extern "C" {

static TransformerConfig config_from_c(const hm_transformer_config *cfg) {
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
    c.eos_token_id = cfg->eos_token_id;
    c.bos_token_id = cfg->bos_token_id;
    return c;
}

hm_model *hm_model_create(hm_ctx *ctx, const hm_transformer_config *cfg, int weight_dtype,
                          int has_qk_norm) {
    if (!ctx) return nullptr;
    if (!cfg) {
        hm_set_error(ctx, HM_ERR_INVALID, "hm_model_create: NULL config");
        return nullptr;
    }
    auto impl = HfModel::create(ctx, config_from_c(cfg), (DType)weight_dtype, has_qk_norm != 0);
    if (!impl) return nullptr;
    return new hm_model{ctx, std::move(impl)};
}

hm_model *hm_model_create_mixed(hm_ctx *ctx, const hm_transformer_config *cfg, const int *proj_dtypes,
                                int has_qk_norm) {
    if (!ctx) return nullptr;
    if (!cfg || !proj_dtypes || cfg->num_hidden_layers <= 0) {
        hm_set_error(ctx, HM_ERR_INVALID, "hm_model_create_mixed: NULL config or dtype list");
        return nullptr;
    }
    std::vector<DType> dts((size_t)cfg->num_hidden_layers * 7);
    for (size_t i = 0; i < dts.size(); i++) {
        if (proj_dtypes[i] < HM_DTYPE_Q8_0 || proj_dtypes[i] > HM_DTYPE_Q6_K || proj_dtypes[i] == HM_DTYPE_I64) {
            hm_set_error(ctx, HM_ERR_INVALID, "hm_model_create_mixed: projection %zu has dtype %d, not a block-quantised one",
                         i, proj_dtypes[i]);
            return nullptr;
        }
        dts[i] = (DType)proj_dtypes[i];
    }
    auto impl = HfModel::create(ctx, config_from_c(cfg), dts[0], has_qk_norm != 0, &dts);
    if (!impl) return nullptr;
    return new hm_model{ctx, std::move(impl)};
}

void hm_model_destroy(hm_model *m) { delete m; }

int hm_model_prefill(hm_model *m, const int64_t *h_ids, int n_ids, float *h_logits) {
    if (!m) return HM_ERR_INVALID;
    return m->impl->prefill(h_ids, n_ids, h_logits);
}

int hm_model_generate(hm_model *m, const int64_t *h_prompt, int n_prompt, int max_new_tokens,
                      const hm_sampling_config *cfg, uint64_t seed, int eos_token_id, int32_t *h_tokens_out,
                      int *n_tokens_out) {
    if (!m) return HM_ERR_INVALID;
    if (!cfg) return hm_set_error(m->ctx, HM_ERR_INVALID, "hm_model_generate: NULL sampling configuration");
    return m->impl->generate(h_prompt, n_prompt, max_new_tokens, *cfg, seed, eos_token_id, h_tokens_out, n_tokens_out);
}

int hm_model_set_prefill_pieces(hm_model *m, int pieces) {
    if (!m) return HM_ERR_INVALID;
    if (pieces != 2 && pieces != 3) return hm_set_error(m->ctx, HM_ERR_INVALID, "prefill pieces must be 2 or 3");
    m->impl->set_prefill_pieces(pieces);
    return HM_OK;
}

int hm_model_set_prefill_weight_cache(hm_model *m, size_t bytes) {
    if (!m) return HM_ERR_INVALID;
    m->impl->set_prefill_weight_cache(bytes);
    return HM_OK;
}

int hm_model_set_prefill_min(hm_model *m, int n_tokens) {
    if (!m || n_tokens < 0) return HM_ERR_INVALID;
    m->impl->set_prefill_min(n_tokens);
    return HM_OK;
}

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

int hm_model_set_weight_nk(hm_model *m, int slot, const void *h_data, size_t bytes) {
    if (!m) return HM_ERR_INVALID;
    return m->impl->set_weight_nk(slot, h_data, bytes);
}

int hm_model_set_lm_head_blocks(hm_model *m, int dtype, const void *h_blocks, size_t bytes) {
    if (!m) return HM_ERR_INVALID;
    if (dtype != HM_DTYPE_Q8_0 && dtype != HM_DTYPE_Q4_0 && dtype != HM_DTYPE_Q4_K && dtype != HM_DTYPE_Q6_K)
        return hm_set_error(m->ctx, HM_ERR_INVALID, "hm_model_set_lm_head_blocks: dtype %d is not a block type", dtype);
    return m->impl->set_lm_head_blocks((DType)dtype, h_blocks, bytes);
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

int hm_model_set_whole_step(hm_model *m, int on) {
    if (!m) return HM_ERR_INVALID;
    return m->impl->set_whole_step(on != 0);
}

int hm_model_whole_step(hm_model *m) {
    if (!m) return HM_ERR_INVALID;
    return m->impl->whole_step() ? 1 : 0;
}

int hm_model_whole_step_available(hm_model *m) {
    if (!m) return HM_ERR_INVALID;
    return m->impl->whole_step_available() ? 1 : 0;
}

int hm_model_prefill_capture_q8k_inputs(hm_model *m, int rows) {
    if (!m) return HM_ERR_INVALID;
    return m->impl->prefill_capture_q8k_inputs(rows);
}

int hm_model_prefill_captured_q8k_inputs(hm_model *m, float *h_out, size_t n_floats) {
    if (!m || !h_out) return HM_ERR_INVALID;
    return m->impl->prefill_captured_q8k_inputs(h_out, n_floats);
}

int hm_model_whole_step_trace(hm_model *m, unsigned long long *h_out, int cap, int *n_out) {
    if (!m || !n_out) return HM_ERR_INVALID;
    return m->impl->whole_step_trace(h_out, cap, n_out);
}

int hm_model_whole_step_inject_timeout(hm_model *m, int workgroup, int spin_limit) {
    if (!m || !m->impl) return HM_ERR_INVALID;
    return m->impl->whole_step_inject_timeout(workgroup, spin_limit);
}

int hm_model_whole_step_status(hm_model *m) {
    if (!m) return HM_ERR_INVALID;
    return m->impl->whole_step_status();
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

// ── checkpoint containers ────────────────────────────────────────────────────

struct hm_gguf {
    std::unique_ptr<GgufFile> f;
};
struct hm_safetensors {
    std::unique_ptr<SafeTensorsFile> f;
};

static void copy_err(const std::string &msg, char *err, size_t errlen) {
    if (err && errlen) snprintf(err, errlen, "%s", msg.c_str());
}

static void fill_c_config(const TransformerConfig &c, hm_transformer_config *out) {
    out->hidden_size = c.hidden_size;
    out->intermediate_size = c.intermediate_size;
    out->num_attention_heads = c.num_attention_heads;
    out->num_hidden_layers = c.num_hidden_layers;
    out->num_key_value_heads = c.num_key_value_heads;
    out->vocab_size = c.vocab_size;
    out->head_dim = c.head_dim_opt;
    out->max_position_embeddings = c.max_position_embeddings;
    out->tie_word_embeddings = c.tie_word_embeddings ? 1 : 0;
    out->rms_norm_eps = c.rms_norm_eps;
    out->rope_theta = c.rope_theta;
    out->attention_bias = c.attention_bias ? 1 : 0;
    out->eos_token_id = c.eos_token_id;
    out->bos_token_id = c.bos_token_id;
}

extern "C" {

hm_gguf *hm_gguf_open(const char *path, char *err, size_t errlen) {
    std::string e;
    auto f = GgufFile::load(path ? path : "", &e);
    if (!f) {
        copy_err(e, err, errlen);
        return nullptr;
    }
    return new hm_gguf{std::move(f)};
}
void hm_gguf_close(hm_gguf *g) { delete g; }
int hm_gguf_version(const hm_gguf *g) { return g ? (int)g->f->version() : HM_ERR_INVALID; }
int hm_gguf_num_tensors(const hm_gguf *g) { return g ? (int)g->f->tensors().size() : HM_ERR_INVALID; }
size_t hm_gguf_data_offset(const hm_gguf *g) { return g ? g->f->data_offset() : 0; }

int hm_gguf_tensor_info(const hm_gguf *g, int index, char *name_buf, size_t buflen, int *n_dims, uint64_t dims[8],
                        int *ggml_type, uint64_t *offset, size_t *nbytes) {
    if (!g || index < 0 || index >= (int)g->f->tensors().size()) return HM_ERR_INVALID;
    const GgufTensorInfo &t = g->f->tensors()[index];
    if (name_buf && buflen) snprintf(name_buf, buflen, "%s", t.name.c_str());
    if (n_dims) *n_dims = (int)t.shape.size();
    if (dims)
        for (size_t i = 0; i < t.shape.size() && i < 8; i++) dims[i] = t.shape[i];
    if (ggml_type) *ggml_type = (int)t.type;
    if (offset) *offset = t.offset;
    if (nbytes) *nbytes = t.byte_size();
    return HM_OK;
}

int hm_gguf_find_tensor(const hm_gguf *g, const char *name) {
    if (!g || !name) return HM_ERR_INVALID;
    const GgufTensorInfo *t = g->f->tensor_info(name);
    return t ? (int)(t - g->f->tensors().data()) : -1;
}

const void *hm_gguf_tensor_data(const hm_gguf *g, int index) {
    if (!g || index < 0 || index >= (int)g->f->tensors().size()) return nullptr;
    return g->f->tensor_data(g->f->tensors()[index]);
}

int hm_gguf_tensor_f32(const hm_gguf *g, int index, float *out, size_t n_elements, char *err, size_t errlen) {
    auto say = [&](const std::string &m) {
        if (err && errlen) snprintf(err, errlen, "%s", m.c_str());
        return HM_ERR_INVALID;
    };
    if (!g || !out || index < 0 || index >= (int)g->f->tensors().size()) return say("bad handle, index or output");
    const GgufTensorInfo &t = g->f->tensors()[index];
    if (t.num_elements() != n_elements)
        return say("tensor " + t.name + " has " + std::to_string(t.num_elements()) + " elements");
    std::vector<float> tmp;
    std::string e;
    if (!ggml_to_f32(t.type, g->f->tensor_data(t), n_elements, &tmp, &e)) return say("tensor " + t.name + ": " + e);
    std::memcpy(out, tmp.data(), n_elements * sizeof(float));
    return HM_OK;
}

int hm_gguf_meta_str(const hm_gguf *g, const char *key, char *buf, size_t buflen) {
    std::string s;
    const GgufValue *v = g && key ? g->f->meta(key) : nullptr;
    if (!v || !v->as_str(&s)) return HM_ERR_INVALID;
    if (buf && buflen) snprintf(buf, buflen, "%s", s.c_str());
    return (int)s.size();
}
int hm_gguf_meta_u64(const hm_gguf *g, const char *key, uint64_t *out) {
    const GgufValue *v = g && key ? g->f->meta(key) : nullptr;
    return v && out && v->as_u64(out) ? HM_OK : HM_ERR_INVALID;
}
int hm_gguf_meta_f32(const hm_gguf *g, const char *key, float *out) {
    const GgufValue *v = g && key ? g->f->meta(key) : nullptr;
    return v && out && v->as_f32(out) ? HM_OK : HM_ERR_INVALID;
}
int64_t hm_gguf_meta_array_len(const hm_gguf *g, const char *key) {
    const GgufValue *v = g && key ? g->f->meta(key) : nullptr;
    return v && v->kind == GgufValue::Array ? (int64_t)v->arr.size() : -1;
}

int hm_gguf_transformer_config(const hm_gguf *g, hm_transformer_config *out, int *has_qk_norm, char *err,
                               size_t errlen) {
    if (!g || !out) return HM_ERR_INVALID;
    TransformerConfig c;
    std::string e;
    if (!g->f->transformer_config(&c, &e)) {
        copy_err(e, err, errlen);
        return HM_ERR_INVALID;
    }
    fill_c_config(c, out);
    if (has_qk_norm) *has_qk_norm = g->f->tensor_info("blk.0.attn_q_norm.weight") != nullptr;
    return HM_OK;
}

hm_safetensors *hm_safetensors_open(const char *path, char *err, size_t errlen) {
    std::string e;
    auto f = SafeTensorsFile::load(path ? path : "", &e);
    if (!f) {
        copy_err(e, err, errlen);
        return nullptr;
    }
    return new hm_safetensors{std::move(f)};
}
void hm_safetensors_close(hm_safetensors *s) { delete s; }
int hm_safetensors_num_tensors(const hm_safetensors *s) { return s ? (int)s->f->tensors().size() : HM_ERR_INVALID; }
int hm_safetensors_tensor_info(const hm_safetensors *s, int index, char *name_buf, size_t buflen, char dtype_buf[8],
                               int *n_dims, uint64_t dims[8], size_t *nbytes) {
    if (!s || index < 0 || index >= (int)s->f->tensors().size()) return HM_ERR_INVALID;
    const SafeTensorInfo &t = s->f->tensors()[index];
    if (name_buf && buflen) snprintf(name_buf, buflen, "%s", t.name.c_str());
    if (dtype_buf) snprintf(dtype_buf, 8, "%s", t.dtype.c_str());
    if (n_dims) *n_dims = (int)t.shape.size();
    if (dims)
        for (size_t i = 0; i < t.shape.size() && i < 8; i++) dims[i] = t.shape[i];
    if (nbytes) *nbytes = t.end - t.begin;
    return HM_OK;
}
const void *hm_safetensors_tensor_data(const hm_safetensors *s, int index) {
    if (!s || index < 0 || index >= (int)s->f->tensors().size()) return nullptr;
    return s->f->data(s->f->tensors()[index]);
}

int hm_config_from_json(const char *json_text, hm_transformer_config *out, char *err, size_t errlen) {
    if (!json_text || !out) return HM_ERR_INVALID;
    TransformerConfig c;
    std::string e;
    if (!transformer_config_from_json(json_text, &c, &e)) {
        copy_err(e, err, errlen);
        return HM_ERR_INVALID;
    }
    fill_c_config(c, out);
    return HM_OK;
}

hm_model *hm_model_load_gguf(hm_ctx *ctx, const char *path, int max_seq_len) {
    if (!ctx || !path) return nullptr;
    auto impl = load_gguf_model(ctx, path, max_seq_len);
    if (!impl) return nullptr;
    return new hm_model{ctx, std::move(impl)};
}

hm_model *hm_model_load_hf_dir(hm_ctx *ctx, const char *dir, int max_seq_len) {
    if (!ctx || !dir) return nullptr;
    auto impl = load_hf_model_dir(ctx, dir, max_seq_len);
    if (!impl) return nullptr;
    return new hm_model{ctx, std::move(impl)};
}

int hm_model_config(hm_model *m, hm_transformer_config *out, int *has_qk_norm, int *weight_dtype) {
    if (!m || !out) return HM_ERR_INVALID;
    fill_c_config(m->impl->config(), out);
    if (has_qk_norm) *has_qk_norm = m->impl->has_qk_norm() ? 1 : 0;
    if (weight_dtype) *weight_dtype = (int)m->impl->weight_dtype();
    return HM_OK;
}

}  // extern "C"
