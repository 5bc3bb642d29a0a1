// HfModel and the bf16 plan emitter on the GPU runtime (see hf.h).
#include "hf.h"

#include <algorithm>
#include <cmath>
#include <cstdlib>

#include "../attention.h"
#include "../decode_fused.h"
#include "../kquant_planes8.h"
#include "../gemm_kquant_i8.h"
#include "../gemv_bf16.h"
#include "../gemm_bf16_mfma.h"
#include "../gemv_k8.h"
#include "../gemv_kquant.h"
#include "../gemv_quant.h"
#include "../gemv_quant_planes.h"
#include "../prefill.h"
#include "../light_ops.h"

namespace homura {

namespace {

// reference precompute_rope_cos_sin (src/hf/precompute.rs:10-40): f64 angle
// pos / theta^(2i/head_dim), rounded to f32, both halves of a row identical.
void precompute_rope_cos_sin(int head_dim, int max_seq_len, double theta, std::vector<float> &cosv,
                             std::vector<float> &sinv) {
    const int half = head_dim / 2;
    cosv.assign((size_t)max_seq_len * head_dim, 0.f);
    sinv.assign((size_t)max_seq_len * head_dim, 0.f);
    for (int pos = 0; pos < max_seq_len; pos++)
        for (int i = 0; i < half; i++) {
            const double freq = 1.0 / std::pow(theta, 2.0 * (double)i / (double)head_dim);
            const double angle = (double)pos * freq;
            const float c = (float)std::cos(angle), s = (float)std::sin(angle);
            cosv[(size_t)pos * head_dim + i] = c;
            cosv[(size_t)pos * head_dim + half + i] = c;
            sinv[(size_t)pos * head_dim + i] = s;
            sinv[(size_t)pos * head_dim + half + i] = s;
        }
}

// HOMURA_WHOLE_STEP_FAR=1 (read when the plan is built): the whole-step kernel takes every exchange through
// memory, as it does when it does not find its workgroups dealt to the dies round-robin.
int whole_step_far_only() {
    const char *e = std::getenv("HOMURA_WHOLE_STEP_FAR");
    return e && std::atoi(e) != 0 ? 1 : 0;
}

}  // namespace

std::unique_ptr<HfModel> HfModel::create(hm_ctx *ctx, const TransformerConfig &cfg,
                                         DType weight_dtype, bool has_qk_norm,
                                         const std::vector<DType> *proj_dtypes) {
    auto fail = [&](const char *msg) -> std::unique_ptr<HfModel> {
        hm_set_error(ctx, HM_ERR_INVALID, "hm_model_create: %s", msg);
        return nullptr;
    };
    if (cfg.hidden_size <= 0 || cfg.intermediate_size <= 0 || cfg.num_attention_heads <= 0 ||
        cfg.num_hidden_layers <= 0 || cfg.vocab_size <= 0)
        return fail("config has a non-positive dimension");
    if (cfg.num_attention_heads % cfg.kv_heads() != 0) return fail("heads not divisible by kv heads");
    if (cfg.head_dim() != 128 && cfg.head_dim() != 64) return fail("head_dim must be 64 or 128");
    if (cfg.gqa_repeat() > 8) return fail("GQA group larger than 8");
    if (cfg.hidden_size % 32 || cfg.intermediate_size % 32 || cfg.q_dim() % 32)
        return fail("hidden, intermediate and q dims must be multiples of 32");
    if (weight_dtype != DType::BF16 && !dtype_is_quantized(weight_dtype))
        return fail("projection dtype must be BF16, Q8_0, Q4_0, Q4_K or Q6_K");
    if (proj_dtypes) {
        if (proj_dtypes->size() != (size_t)cfg.num_hidden_layers * 7) return fail("need 7 projection dtypes per layer");
        for (DType t : *proj_dtypes)
            if (!dtype_is_quantized(t)) return fail("a model with per-projection dtypes must be quantised throughout");
        if (!dtype_is_quantized(weight_dtype)) return fail("per-projection dtypes need a quantised weight_dtype");
    }

    std::unique_ptr<HfModel> m(new HfModel());
    m->ctx_ = ctx;
    m->cfg_ = cfg;
    m->weight_dtype_ = weight_dtype;
    m->proj_dtypes_ = proj_dtypes ? *proj_dtypes : std::vector<DType>((size_t)cfg.num_hidden_layers * 7, weight_dtype);
    if (dtype_is_quantized(weight_dtype)) {
        const int kdim[7] = {cfg.hidden_size, cfg.hidden_size, cfg.hidden_size, cfg.q_dim(), cfg.hidden_size,
                             cfg.hidden_size, cfg.intermediate_size};
        for (size_t i = 0; i < m->proj_dtypes_.size(); i++)
            if (kdim[i % 7] % (int)dtype_block_size(m->proj_dtypes_[i]) != 0)
                return fail("a projection's input width is not a multiple of its quantisation block");
    }
    m->has_qk_norm_ = has_qk_norm;

    // Slot order = TransformerWeights::to_slot_buffers (src/hf/weights.rs:63-116) for bf16,
    // to_slot_buffers_quant (:136-183) for block-quantised projections.
    const int64_t hidden = cfg.hidden_size, inter = cfg.intermediate_size, vocab = cfg.vocab_size;
    const int64_t qd = cfg.q_dim(), kvd = cfg.kv_dim(), hd = cfg.head_dim();
    const bool quant = dtype_is_quantized(weight_dtype);
    auto &v = m->infos_;
    auto f32_vec = [&](const std::string &name, int64_t n) {
        v.push_back(WeightSlotInfo{name, DType::F32, n, 1, (size_t)n * 4});
    };
    int proj_index = 0;  // runs over (layer, q k v o gate up down) in slot order
    auto proj = [&](const std::string &name, int64_t K, int64_t N) {
        if (quant) {
            const DType t = m->proj_dtypes_[proj_index++];
            v.push_back(WeightSlotInfo{name, t, N, K, dtype_bytes_for_elements(t, (size_t)(N * K), nullptr)});
        } else
            v.push_back(WeightSlotInfo{name, DType::BF16, K, N, (size_t)(K * N) * 2});
    };
    v.push_back(WeightSlotInfo{"model.embed_tokens.weight", DType::F32, vocab, hidden,
                               (size_t)(vocab * hidden) * 4});
    for (int l = 0; l < cfg.num_hidden_layers; l++) {
        const std::string p = "model.layers." + std::to_string(l) + ".";
        f32_vec(p + "input_layernorm.weight", hidden);
        proj(p + "self_attn.q_proj.weight", hidden, qd);
        if (cfg.attention_bias) f32_vec(p + "self_attn.q_proj.bias", qd);
        proj(p + "self_attn.k_proj.weight", hidden, kvd);
        if (cfg.attention_bias) f32_vec(p + "self_attn.k_proj.bias", kvd);
        proj(p + "self_attn.v_proj.weight", hidden, kvd);
        if (cfg.attention_bias) f32_vec(p + "self_attn.v_proj.bias", kvd);
        if (has_qk_norm) {
            f32_vec(p + "self_attn.q_norm.weight", hd);
            f32_vec(p + "self_attn.k_norm.weight", hd);
        }
        proj(p + "self_attn.o_proj.weight", qd, hidden);
        f32_vec(p + "post_attention_layernorm.weight", hidden);
        proj(p + "mlp.gate_proj.weight", hidden, inter);
        proj(p + "mlp.up_proj.weight", hidden, inter);
        proj(p + "mlp.down_proj.weight", inter, hidden);
    }
    f32_vec("model.norm.weight", hidden);
    if (quant)  // the quantised plan keeps the LM head in f32 (src/hf/weights.rs:174-180)
        v.push_back(WeightSlotInfo{"lm_head.weight", DType::F32, hidden, vocab, (size_t)(hidden * vocab) * 4});
    else
        v.push_back(WeightSlotInfo{"lm_head.weight", DType::BF16, hidden, vocab, (size_t)(hidden * vocab) * 2});

    for (size_t i = 0; i < v.size(); i++) m->slot_by_name_[v[i].name] = (int)i;
    m->weight_bufs_.resize(v.size());
    m->weight_set_.assign(v.size(), false);
    m->packed_.resize(cfg.num_hidden_layers);
    return m;
}

void HfModel::quant_run(int layer, int which, int *first, int *count) const {
    int lo = which, hi = which;  // q|k|v are 0..2, gate|up are 4..5; o and down stand alone
    const int gmin = which <= 2 ? 0 : which == 4 || which == 5 ? 4 : which;
    const int gmax = which <= 2 ? 2 : which == 4 || which == 5 ? 5 : which;
    const DType t = proj_dtype(layer, which);
    while (lo > gmin && proj_dtype(layer, lo - 1) == t) lo--;
    while (hi < gmax && proj_dtype(layer, hi + 1) == t) hi++;
    *first = lo;
    *count = hi - lo + 1;
}

// The decode GEMVs of Q8_0 / Q4_0 runs read a re-packed copy of the blocks (quant bytes and scales in
// planes of their own: same bytes, naturally aligned words); the raw blocks stay for the prompt pass and
// the weight listing. HOMURA_QUANT_PLANES=0 keeps the decode on the raw blocks.
int HfModel::build_quant_planes() {
    if (const char *e = std::getenv("HOMURA_QUANT_PLANES"))
        if (std::atoi(e) == 0) return HM_OK;
    const int hidden = cfg_.hidden_size, inter = cfg_.intermediate_size, qd = cfg_.q_dim(), kvd = cfg_.kv_dim();
    const int kdim[7] = {hidden, hidden, hidden, qd, hidden, hidden, inter};
    const int ndim[7] = {qd, kvd, kvd, hidden, inter, inter, hidden};
    for (int l = 0; l < cfg_.num_hidden_layers; l++)
        for (int j = 0; j < 7; j++) {
            int first, count;
            quant_run(l, j, &first, &count);
            const DType t = proj_dtype(l, j);
            if (first != j || (t != DType::Q8_0 && t != DType::Q4_0) || kdim[j] > 16384 || !packed_[l].quant[j]) continue;
            int n = 0;
            for (int e = j; e < j + count; e++) n += ndim[e];
            const size_t bytes = quant_planes_bytes(t == DType::Q4_0, n, kdim[j]);
            packed_[l].planes[j] = Buffer::alloc_bytes(ctx_, bytes, {(int64_t)bytes}, t);
            if (!packed_[l].planes[j]) return HM_ERR_OOM;
            const int rc = pack_quant_planes(ctx_, t == DType::Q4_0, packed_[l].quant[j].as<uint8_t>(),
                                             packed_[l].planes[j].as<uint8_t>(), n, kdim[j]);
            if (rc != HM_OK) return rc;
        }
    if (lm_head_blocks_ && (lm_head_blocks_dtype_ == DType::Q8_0 || lm_head_blocks_dtype_ == DType::Q4_0) && hidden <= 4096) {
        const bool q4 = lm_head_blocks_dtype_ == DType::Q4_0;
        const size_t bytes = quant_planes_bytes(q4, cfg_.vocab_size, hidden);
        lm_head_planes_ = Buffer::alloc_bytes(ctx_, bytes, {(int64_t)bytes}, lm_head_blocks_dtype_);
        if (!lm_head_planes_) return HM_ERR_OOM;
        const int rc = pack_quant_planes(ctx_, q4, lm_head_blocks_.as<uint8_t>(), lm_head_planes_.as<uint8_t>(), cfg_.vocab_size, hidden);
        if (rc != HM_OK) return rc;
    }
    if (lm_head_blocks_ && lm_head_blocks_dtype_ == DType::Q6_K && q6k_planes_shape_ok(cfg_.vocab_size, hidden)) {
        const size_t bytes = q6k_planes_bytes(cfg_.vocab_size, hidden);
        lm_head_planes_ = Buffer::alloc_bytes(ctx_, bytes, {(int64_t)bytes}, lm_head_blocks_dtype_);
        if (!lm_head_planes_) return HM_ERR_OOM;
        const int rc = pack_q6k_planes(ctx_, lm_head_blocks_.as<uint8_t>(), lm_head_planes_.as<uint8_t>(), cfg_.vocab_size, hidden, false);
        if (rc != HM_OK) return rc;
    }
    return hm_sync(ctx_);
}

// A model whose projections are all Q4_K or Q6_K (the Q4_K_M-style mixes): every group of matrices that share an
// activation (q|k|v, o, gate|up, down) once more as byte planes with per-row scale records, which the whole-step
// launch reads (the raw blocks stay for the prompt pass, the per-projection path and the weight listing).
int HfModel::build_k8_planes() {
    const int hidden = cfg_.hidden_size, inter = cfg_.intermediate_size, qd = cfg_.q_dim(), kvd = cfg_.kv_dim();
    const int kdim[7] = {hidden, hidden, hidden, qd, hidden, hidden, inter};
    const int ndim[7] = {qd, kvd, kvd, hidden, inter, inter, hidden};
    const int group_first[4] = {0, 3, 4, 6}, group_count[4] = {3, 1, 2, 1};
    for (int l = 0; l < cfg_.num_hidden_layers; l++)
        for (int g = 0; g < 4; g++) {
            const int K = kdim[group_first[g]];
            int n = 0;
            for (int e = 0; e < group_count[g]; e++) n += ndim[group_first[g] + e];
            const size_t bytes = k8_plane_bytes(n, K) + k8_record_bytes(n, K);
            Buffer &dst = packed_[l].k8[g];
            dst = Buffer::alloc_bytes(ctx_, bytes, {(int64_t)bytes}, DType::Q4_K);
            if (!dst) return HM_ERR_OOM;
            int row0 = 0;
            for (int e = 0; e < group_count[g]; e++) {
                const int j = group_first[g] + e;
                const DType t = proj_dtype(l, j);
                // projection j's raw blocks sit in the run of same-typed neighbours that starts at `first`
                int first, count;
                quant_run(l, j, &first, &count);
                if (!packed_[l].quant[first]) return hm_set_error(ctx_, HM_ERR_STATE, "layer %d projection %d has no blocks", l, j);
                size_t skip = 0;
                for (int b = first; b < j; b++) skip += dtype_bytes_for_elements(t, (size_t)ndim[b] * K, nullptr);
                const bool pairs = k8_pairs_ && g == 2;  // gate row r -> 2 r, up row r -> 2 r + 1
                const int rc = pack_k8_rows(ctx_, t == DType::Q6_K ? HM_DTYPE_Q6_K : HM_DTYPE_Q4_K,
                                            packed_[l].quant[first].as<uint8_t>() + skip, ndim[j], K, dst.as<uint8_t>(),
                                            dst.as<uint8_t>() + k8_plane_bytes(n, K), pairs ? e : row0, pairs ? 2 : 1);
                if (rc != HM_OK) return rc;
                row0 += ndim[j];
            }
        }
    return hm_sync(ctx_);
}

HfModel::~HfModel() {
    if (ctx_) hm_sync(ctx_);
    if (h_stage_) (void)hipHostFree(h_stage_);
}

int HfModel::set_weight_impl(int slot, const void *h_data, size_t bytes, bool nk_layout) {
    if (slot < 0 || slot >= (int)infos_.size())
        return hm_set_error(ctx_, HM_ERR_INVALID, "weight slot %d out of range (have %zu)", slot, infos_.size());
    const WeightSlotInfo &info = infos_[slot];
    if (bytes != info.bytes)  // the reference panics on a weight byte-size mismatch
                              // (src/hf/emitter_quant.rs:1462-1478)
        return hm_set_error(ctx_, HM_ERR_INVALID, "weight %s: expected %zu bytes, got %zu",
                            info.name.c_str(), info.bytes, bytes);
    if (finalized_) return hm_set_error(ctx_, HM_ERR_STATE, "model already finalized");
    if (!h_data) return hm_set_error(ctx_, HM_ERR_INVALID, "weight %s: NULL data", info.name.c_str());

    const std::string &nm = info.name;
    auto ends_with = [&](const char *suffix) {
        const std::string s(suffix);
        return nm.size() >= s.size() && nm.compare(nm.size() - s.size(), s.size(), s) == 0;
    };
    const int hidden = cfg_.hidden_size, inter = cfg_.intermediate_size;
    const int qd = cfg_.q_dim(), kvd = cfg_.kv_dim();

    if (dtype_is_quantized(info.dtype)) {
        // Raw GGUF blocks [N][K/block], kept byte for byte. Neighbours of one type inside q|k|v and
        // gate|up of a layer are stored back to back (rows are contiguous, so the matrices form
        // one taller matrix and one kernel launch serves them).
        const size_t p0 = std::string("model.layers.").size();
        const int layer = std::atoi(nm.c_str() + p0);
        LayerPacked &lp = packed_[layer];
        static const char *const suffix[7] = {"q_proj.weight", "k_proj.weight", "v_proj.weight", "o_proj.weight",
                                              "gate_proj.weight", "up_proj.weight", "down_proj.weight"};
        int which = -1;
        for (int j = 0; j < 7; j++)
            if (ends_with(suffix[j])) which = j;
        if (which < 0) return hm_set_error(ctx_, HM_ERR_INVALID, "unexpected quantised weight %s", nm.c_str());
        const int64_t kdim[7] = {hidden, hidden, hidden, qd, hidden, hidden, inter};
        const int64_t ndim[7] = {qd, kvd, kvd, hidden, inter, inter, hidden};
        int first, count;
        quant_run(layer, which, &first, &count);
        size_t home_bytes = 0, offset = 0;
        for (int j = first; j < first + count; j++) {
            const size_t b = dtype_bytes_for_elements(info.dtype, (size_t)(kdim[j] * ndim[j]), nullptr);
            if (j < which) offset += b;
            home_bytes += b;
        }
        Buffer *home = &lp.quant[first];
        if (!*home) *home = Buffer::alloc_bytes(ctx_, home_bytes, {(int64_t)home_bytes}, info.dtype);
        if (!*home) return HM_ERR_OOM;
        int rc = hm_upload(ctx_, (char *)home->ptr() + offset, h_data, bytes);
        if (rc != HM_OK) return rc;
        weight_bufs_[slot] = Buffer::view((char *)home->ptr() + offset, bytes, {(int64_t)bytes}, {1}, info.dtype);
        weight_set_[slot] = true;
        return HM_OK;
    }

    if (info.dtype == DType::F32 && nm == "lm_head.weight") {
        // f32 LM head of the quantised plan: [hidden][vocab] -> [vocab][hidden] stream layout
        lm_head_packed_ = Buffer::alloc(ctx_, {info.dim1, info.dim0}, DType::F32);
        if (!lm_head_packed_) return HM_ERR_OOM;
        int rc;
        if (nk_layout) {
            rc = hm_upload(ctx_, lm_head_packed_.ptr(), h_data, bytes);
        } else {
            Buffer staging = Buffer::alloc_bytes(ctx_, bytes, {info.dim0, info.dim1}, DType::F32);
            if (!staging) return HM_ERR_OOM;
            rc = hm_upload(ctx_, staging.ptr(), h_data, bytes);
            if (rc == HM_OK) rc = pack_f32_kn_to_nk(ctx_, staging.as<float>(), lm_head_packed_.as<float>(),
                                                    (int)info.dim0, (int)info.dim1);
            if (rc == HM_OK) rc = hm_sync(ctx_);
        }
        if (rc != HM_OK) return rc;
        weight_bufs_[slot] = Buffer::view(lm_head_packed_.ptr(), bytes, {info.dim1, info.dim0},
                                          {info.dim0, 1}, DType::F32);
        weight_set_[slot] = true;
        return HM_OK;
    }

    if (ends_with("_proj.bias")) {
        // q|k|v biases of a layer sit back to back like the rows they belong to
        const size_t p0 = std::string("model.layers.").size();
        LayerPacked &lp = packed_[std::atoi(nm.c_str() + p0)];
        if (!lp.qkv_bias) lp.qkv_bias = Buffer::alloc(ctx_, {qd + 2 * kvd}, DType::F32);
        if (!lp.qkv_bias) return HM_ERR_OOM;
        const size_t off = ends_with("q_proj.bias") ? 0 : ends_with("k_proj.bias") ? (size_t)qd : (size_t)(qd + kvd);
        float *dst = lp.qkv_bias.as<float>() + off;
        int rc = hm_upload(ctx_, dst, h_data, bytes);
        if (rc != HM_OK) return rc;
        weight_bufs_[slot] = Buffer::view(dst, bytes, {info.dim0}, {1}, DType::F32);
        weight_set_[slot] = true;
        return HM_OK;
    }

    if (info.dtype != DType::BF16) {
        // f32 vectors and the embedding table are stored as they come
        Buffer b = Buffer::alloc_bytes(ctx_, bytes, {info.dim0, info.dim1}, info.dtype);
        if (!b) return HM_ERR_OOM;
        int rc = hm_upload(ctx_, b.ptr(), h_data, bytes);
        if (rc != HM_OK) return rc;
        weight_bufs_[slot] = std::move(b);
        weight_set_[slot] = true;
        return HM_OK;
    }

    // bf16 projection [K][N]: stage, then transpose into its place in the packed stream buffers
    // ([N][K] input goes there as it is)
    const int K = (int)info.dim0, N = (int)info.dim1;
    Buffer staging;
    int rc = HM_OK;
    if (!nk_layout) {
        staging = Buffer::alloc_bytes(ctx_, bytes, {K, N}, DType::BF16);
        if (!staging) return HM_ERR_OOM;
        rc = hm_upload(ctx_, staging.ptr(), h_data, bytes);
        if (rc != HM_OK) return rc;
    }

    uint16_t *dst = nullptr;
    int row_mult = 1, row_off = 0;
    auto ensure = [&](Buffer &b, int64_t rows, int64_t cols) -> bool {
        if (!b) b = Buffer::alloc(ctx_, {rows, cols}, DType::BF16);
        return (bool)b;
    };
    if (nm == "lm_head.weight") {
        if (!ensure(lm_head_packed_, cfg_.vocab_size, hidden)) return HM_ERR_OOM;
        dst = lm_head_packed_.as<uint16_t>();
    } else {
        const size_t p0 = std::string("model.layers.").size();
        const int layer = std::atoi(nm.c_str() + p0);
        LayerPacked &lp = packed_[layer];
        if (ends_with("q_proj.weight") || ends_with("k_proj.weight") || ends_with("v_proj.weight")) {
            if (!ensure(lp.qkv, qd + 2 * kvd, hidden)) return HM_ERR_OOM;
            const size_t row0 = ends_with("q_proj.weight") ? 0 : ends_with("k_proj.weight") ? qd : qd + kvd;
            dst = lp.qkv.as<uint16_t>() + row0 * hidden;
        } else if (ends_with("o_proj.weight")) {
            if (!ensure(lp.o, hidden, qd)) return HM_ERR_OOM;
            dst = lp.o.as<uint16_t>();
        } else if (ends_with("gate_proj.weight") || ends_with("up_proj.weight")) {
            // rows interleaved (gate_0, up_0, gate_1, up_1, ...) so one wavefront finishes
            // silu(gate_i) * up_i without a second pass
            if (!ensure(lp.gate_up, 2 * (int64_t)inter, hidden)) return HM_ERR_OOM;
            dst = lp.gate_up.as<uint16_t>();
            row_mult = 2;
            row_off = ends_with("up_proj.weight") ? 1 : 0;
        } else if (ends_with("down_proj.weight")) {
            if (!ensure(lp.down, hidden, inter)) return HM_ERR_OOM;
            dst = lp.down.as<uint16_t>();
        } else {
            return hm_set_error(ctx_, HM_ERR_INVALID, "unexpected bf16 weight %s", nm.c_str());
        }
    }
    if (nk_layout) {
        HM_HIP(ctx_, hipMemcpy2DAsync(dst + (size_t)row_off * K, (size_t)K * 2 * row_mult, h_data, (size_t)K * 2,
                                      (size_t)K * 2, (size_t)N, hipMemcpyHostToDevice, ctx_->stream));
    } else {
        rc = pack_bf16_kn_to_nk_strided(ctx_, staging.as<uint16_t>(), dst, K, N, row_mult, row_off);
        if (rc != HM_OK) return rc;
    }
    if ((rc = hm_sync(ctx_)) != HM_OK) return rc;
    // the slot buffer is a view of the packed rows ([N][K], K contiguous; interleaved slots
    // have a doubled row stride)
    weight_bufs_[slot] = Buffer::view(dst + (size_t)row_off * K, (size_t)N * K * 2 * row_mult, {N, K},
                                      {(int64_t)K * row_mult, 1}, DType::BF16);
    weight_set_[slot] = true;
    return HM_OK;
}

int HfModel::set_lm_head_blocks(DType dtype, const void *h_blocks, size_t bytes) {
    if (finalized_) return hm_set_error(ctx_, HM_ERR_STATE, "set_lm_head_blocks after finalize");
    if (!dtype_is_quantized(weight_dtype_))
        return hm_set_error(ctx_, HM_ERR_INVALID, "set_lm_head_blocks: only block-quantised plans keep an f32 LM head");
    if (!dtype_is_quantized(dtype))
        return hm_set_error(ctx_, HM_ERR_INVALID, "set_lm_head_blocks: Q8_0, Q4_0, Q4_K or Q6_K blocks expected");
    const int64_t hidden = cfg_.hidden_size, vocab = cfg_.vocab_size;
    const int64_t per_block = (dtype == DType::Q4_K || dtype == DType::Q6_K) ? 256 : 32;
    if (hidden % per_block != 0 || hidden > 4096)
        return hm_set_error(ctx_, HM_ERR_INVALID, "set_lm_head_blocks: hidden_size %lld must be a multiple of %lld, at most 4096",
                            (long long)hidden, (long long)per_block);
    size_t want = 0;
    const size_t per = dtype_bytes_for_elements(dtype, (size_t)(hidden * vocab), nullptr);
    want = per;
    if (!h_blocks || bytes != want)
        return hm_set_error(ctx_, HM_ERR_INVALID, "set_lm_head_blocks: %zu bytes given, [%lld][%lld / %lld] blocks take %zu",
                            bytes, (long long)vocab, (long long)hidden, (long long)per_block, want);
    int slot = -1;
    for (size_t i = 0; i < infos_.size(); i++)
        if (infos_[i].name == "lm_head.weight") slot = (int)i;
    if (slot < 0) return hm_set_error(ctx_, HM_ERR_STATE, "set_lm_head_blocks: the plan has no LM head slot");
    lm_head_blocks_ = Buffer::alloc_bytes(ctx_, bytes, {(int64_t)bytes}, dtype);
    if (!lm_head_blocks_) return HM_ERR_OOM;
    const int rc = hm_upload(ctx_, lm_head_blocks_.ptr(), h_blocks, bytes);
    if (rc != HM_OK) return rc;
    lm_head_blocks_dtype_ = dtype;
    lm_head_packed_ = Buffer();  // an f32 head uploaded earlier is no longer needed
    weight_bufs_[slot] = Buffer::view(lm_head_blocks_.ptr(), bytes, {(int64_t)bytes}, {1}, dtype);
    weight_set_[slot] = true;
    return HM_OK;
}

int HfModel::finalize(int max_seq_len) {
    if (finalized_) return HM_OK;
    for (size_t i = 0; i < weight_set_.size(); i++)
        if (!weight_set_[i])  // reference: "missing weight: {key}" (src/hf/weights.rs:276-282)
            return hm_set_error(ctx_, HM_ERR_STATE, "missing weight: %s", infos_[i].name.c_str());
    if (max_seq_len <= 0 || max_seq_len > cfg_.max_position_embeddings)
        return hm_set_error(ctx_, HM_ERR_INVALID, "max_seq_len %d outside 1..max_position_embeddings=%d",
                            max_seq_len, cfg_.max_position_embeddings);
    max_seq_len_ = max_seq_len;

    std::vector<float> cosv, sinv;
    precompute_rope_cos_sin(cfg_.head_dim(), cfg_.max_position_embeddings, cfg_.rope_theta, cosv, sinv);
    rope_cos_ = Buffer::alloc(ctx_, {cfg_.max_position_embeddings, cfg_.head_dim()}, DType::F32);
    rope_sin_ = Buffer::alloc(ctx_, {cfg_.max_position_embeddings, cfg_.head_dim()}, DType::F32);
    if (!rope_cos_ || !rope_sin_) return HM_ERR_OOM;
    int rc = hm_upload(ctx_, rope_cos_.ptr(), cosv.data(), cosv.size() * 4);
    if (rc == HM_OK) rc = hm_upload(ctx_, rope_sin_.ptr(), sinv.data(), sinv.size() * 4);
    if (rc != HM_OK) return rc;

    scratch_ = std::make_shared<PlanScratch>();
    PlanScratch &s = *scratch_;
    s.attn_flat = Buffer::alloc(ctx_, {cfg_.q_dim()}, DType::F32);
    s.resid = Buffer::alloc(ctx_, {cfg_.hidden_size}, DType::F32);
    s.act = Buffer::alloc(ctx_, {cfg_.intermediate_size}, DType::F32);
    s.cand_cap = 4096;
    s.cand_val = Buffer::alloc(ctx_, {s.cand_cap}, DType::F32);
    s.cand_idx = Buffer::alloc(ctx_, {s.cand_cap}, DType::F32);
    if (!s.attn_flat || !s.resid || !s.act || !s.cand_val || !s.cand_idx) return HM_ERR_OOM;

    if (dtype_is_quantized(weight_dtype_) && (rc = build_quant_planes()) != HM_OK) return rc;

    // The whole-step decode launch serves bf16 models, and models whose projections are all Q8_0 or all
    // Q4_0 (re-packed into planes), of a shape it has an instance for.
    fused_available_ = false;
    fused_wf_ = FUSED_WF_BF16;
    bool fused_format = weight_dtype_ == DType::BF16;
    if (dtype_is_quantized(weight_dtype_)) {
        const DType t = proj_dtype(0, 0);
        fused_format = t == DType::Q8_0 || t == DType::Q4_0;
        bool all_kquant = true;  // any mix of Q4_K and Q6_K
        for (int l = 0; l < cfg_.num_hidden_layers; l++)
            for (int j = 0; j < 7; j++) all_kquant = all_kquant && (proj_dtype(l, j) == DType::Q4_K || proj_dtype(l, j) == DType::Q6_K);
        for (int l = 0; l < cfg_.num_hidden_layers && fused_format; l++) {
            for (int j = 0; j < 7; j++) fused_format = fused_format && proj_dtype(l, j) == t;
            fused_format = fused_format && packed_[l].planes[0] && packed_[l].planes[3] && packed_[l].planes[4] && packed_[l].planes[6];
        }
        fused_wf_ = t == DType::Q4_0 ? FUSED_WF_Q4_0 : FUSED_WF_Q8_0;
        if (all_kquant) {
            fused_format = true;
            fused_wf_ = FUSED_WF_K8;
            // the K8 form serves the whole-step launch and the per-projection decode GEMVs alike
            if (cfg_.hidden_size % 256 == 0 && cfg_.q_dim() % 256 == 0 && cfg_.intermediate_size % 256 == 0 &&
                std::max({cfg_.hidden_size, cfg_.q_dim(), cfg_.intermediate_size}) <= 16384) {
                const FusedShape fs8{cfg_.hidden_size, cfg_.num_attention_heads, cfg_.kv_heads(), cfg_.head_dim(),
                                     cfg_.intermediate_size, FUSED_WF_K8};
                k8_pairs_ = !decode_fused_supported(ctx_, fs8, cfg_.num_hidden_layers, max_seq_len, nullptr);
                if ((rc = build_k8_planes()) != HM_OK) return rc;
            }
        }
    }
    if (fused_format) {
        const FusedShape fs{cfg_.hidden_size, cfg_.num_attention_heads, cfg_.kv_heads(), cfg_.head_dim(),
                            cfg_.intermediate_size, fused_wf_};
        bool served = decode_fused_supported(ctx_, fs, cfg_.num_hidden_layers, max_seq_len, nullptr);
        served = served && (fused_wf_ != FUSED_WF_K8 || (bool)packed_[0].k8[0]);
        if (served) {
            s.fused_layers = Buffer::alloc_bytes(ctx_, sizeof(FusedLayerPtrs) * (size_t)cfg_.num_hidden_layers,
                                                 {cfg_.num_hidden_layers}, DType::I64);
            const size_t xb = decode_fused_xch_bytes(fs);
            s.fused_xch = Buffer::alloc_bytes(ctx_, xb, {(int64_t)xb}, DType::I64);
            s.fused_ctl = Buffer::alloc_bytes(ctx_, 64, {16}, DType::I64);
            if (!s.fused_layers || !s.fused_xch || !s.fused_ctl) return HM_ERR_OOM;
            HM_HIP(ctx_, hipMemsetAsync(s.fused_xch.ptr(), 0, xb, ctx_->stream));
            HM_HIP(ctx_, hipMemsetAsync(s.fused_ctl.ptr(), 0, 64, ctx_->stream));
            fused_available_ = true;
        }
    }

    rc = dtype_is_quantized(weight_dtype_) ? emit_transformer_plan_quant() : emit_transformer_plan();
    if (rc != HM_OK) return rc;
    rc = plan_->prepare(std::max(max_seq_len, 16));
    if (rc != HM_OK) return rc;
    rc = plan_->ensure_kv_cache(max_seq_len_);
    if (rc != HM_OK) return rc;
    const FusedShape fs{cfg_.hidden_size, cfg_.num_attention_heads, cfg_.kv_heads(), cfg_.head_dim(),
                        cfg_.intermediate_size, fused_wf_};
    if (fused_available_) {
        fused_max_kv_ = decode_fused_max_kv(fs);
        const char *e = std::getenv("HOMURA_WHOLE_STEP");  // 0: keep one launch per projection
        whole_step_wanted_ = !(e && std::atoi(e) == 0);
    }
    // Before every step: the whole-step launch while the step's live rows (the cache and the new row) are
    // within what its attention phase holds, one launch per projection beyond (a longer conversation
    // changes over once; a cache reset changes back). With one launch per projection the attention grid of the
    // recorded step covers the live rows rounded up to a power of two (2048 at least) instead of the cache's
    // capacity: a cache sized for 32768 rows with 1000 in it would otherwise start 30 workgroups that leave at
    // once for every one that works, and fold its few partial results with the workgroup meant for hundreds.
    plan_->set_pre_run([this, fs]() {
        const int live = plan_->kv_cache_len() + 1;
        int rc = HM_OK;
        if (fused_available_) {
            const int tier = decode_fused_tier(fs, live);  // 0: no instance holds that many rows
            rc = plan_->set_whole_step(whole_step_wanted_ && !fused_gave_up_ && tier > 0);
            fused_dirty_ = fused_dirty_ || plan_->whole_step();
            if (rc == HM_OK && plan_->whole_step() && tier != fused_tier_) {
                rc = plan_->invalidate_graph();  // the recorded launch is another instance's
                fused_tier_ = tier;
            }
            if (rc == HM_OK) rc = refresh_fused_table();
        }
        if (rc == HM_OK && !plan_->whole_step()) {
            int span = 2048;
            while (span < live && span < max_seq_len_) span *= 2;
            span = std::min(span, max_seq_len_);
            if (span != plan_->attn_span()) {
                plan_->set_attn_span(span);
                rc = plan_->invalidate_graph();  // the recorded grids cover the old span
            }
        }
        return rc;
    });
    if (fused_available_ && whole_step_wanted_ && (rc = plan_->set_whole_step(true)) != HM_OK) return rc;
    ids_view_ = Buffer::view(plan_->forced_ids(), (size_t)plan_->out_capacity() * 4, {1, DIM_DYNAMIC},
                             {1, 1}, DType::I64);
    mask_view_ = Buffer::view(plan_->state(), sizeof(DecodeState), {1, 1, 1, DIM_DYNAMIC}, {1, 1, 1, 1},
                              DType::F32);
    finalized_ = true;
    return hm_sync(ctx_);
}

// ── bf16 plan ────────────────────────────────────────────────────────────────
// Slot order and step list follow assign_transformer_slots / emit_transformer_plan
// (reference src/hf/emitter.rs:74-498, :902-1014).
int HfModel::emit_transformer_plan() {
    const TransformerConfig c = cfg_;
    const int64_t hidden = c.hidden_size, inter = c.intermediate_size, vocab = c.vocab_size;
    const int64_t H = c.num_attention_heads, kvh = c.kv_heads(), hd = c.head_dim();
    const int64_t qd = c.q_dim(), kvd = c.kv_dim();
    const int L = c.num_hidden_layers;
    const float eps = (float)c.rms_norm_eps;
    const bool qkn = has_qk_norm_;
    const int64_t D = DIM_DYNAMIC;

    std::vector<SlotDesc> descs;
    auto alloc = [&](std::vector<int64_t> shape, DType dt, const std::string &name) -> size_t {
        descs.push_back(SlotDesc{std::move(shape), dt, name});
        return descs.size() - 1;
    };
    std::vector<size_t> input_slots, weight_slots, past_kv, present_kv;

    const size_t input_ids = alloc({1, D}, DType::I64, "input_ids");
    const size_t mask = alloc({1, 1, D, D}, DType::F32, "mask");
    const size_t cos_s = alloc({D, hd}, DType::F32, "cos");
    const size_t sin_s = alloc({D, hd}, DType::F32, "sin");
    input_slots = {input_ids, mask, cos_s, sin_s};
    const size_t embed_w = alloc({vocab, hidden}, DType::F32, "embed_tokens");
    weight_slots.push_back(embed_w);
    const size_t embed_out = alloc({1, D, hidden}, DType::F32, "embed_out");

    struct LayerSlots {
        size_t hidden_in, input_ln, q_w, k_w, v_w, q_b, k_b, v_b, q_norm, k_norm, o_w, post_ln, gate_w, up_w, down_w;
        size_t q, k, v, past_k, past_v, present_k, present_v, attn_out, hidden_out;
    };
    std::vector<LayerSlots> ls(L);
    for (int i = 0; i < L; i++) {
        LayerSlots &s = ls[i];
        const std::string p = "l" + std::to_string(i) + ".";
        s.hidden_in = i == 0 ? embed_out : ls[i - 1].hidden_out;
        auto w = [&](std::vector<int64_t> shape, DType dt, const std::string &n) {
            size_t slot = alloc(std::move(shape), dt, p + n);
            weight_slots.push_back(slot);
            return slot;
        };
        s.input_ln = w({hidden}, DType::F32, "input_ln");
        const bool bias = c.attention_bias;
        s.q_b = s.k_b = s.v_b = (size_t)-1;
        s.q_w = w({hidden, qd}, DType::BF16, "q_w");
        if (bias) s.q_b = w({qd}, DType::F32, "q_b");
        s.k_w = w({hidden, kvd}, DType::BF16, "k_w");
        if (bias) s.k_b = w({kvd}, DType::F32, "k_b");
        s.v_w = w({hidden, kvd}, DType::BF16, "v_w");
        if (bias) s.v_b = w({kvd}, DType::F32, "v_b");
        s.q_norm = s.k_norm = (size_t)-1;
        if (qkn) {
            s.q_norm = w({hd}, DType::F32, "q_norm");
            s.k_norm = w({hd}, DType::F32, "k_norm");
        }
        s.o_w = w({qd, hidden}, DType::BF16, "o_w");
        s.post_ln = w({hidden}, DType::F32, "post_ln");
        s.gate_w = w({hidden, inter}, DType::BF16, "gate_w");
        s.up_w = w({hidden, inter}, DType::BF16, "up_w");
        s.down_w = w({inter, hidden}, DType::BF16, "down_w");
        s.q = alloc({1, D, H, hd}, DType::F32, p + "q");
        s.k = alloc({1, kvh, D, hd}, DType::F32, p + "k");
        s.v = alloc({1, kvh, D, hd}, DType::F32, p + "v");
        s.past_k = alloc({1, kvh, D, hd}, DType::BF16, p + "past_k");
        s.past_v = alloc({1, kvh, D, hd}, DType::BF16, p + "past_v");
        past_kv.push_back(s.past_k);
        past_kv.push_back(s.past_v);
        input_slots.push_back(s.past_k);
        input_slots.push_back(s.past_v);
        s.present_k = alloc({1, kvh, D, hd}, DType::BF16, p + "present_k");
        s.present_v = alloc({1, kvh, D, hd}, DType::BF16, p + "present_v");
        present_kv.push_back(s.present_k);
        present_kv.push_back(s.present_v);
        s.attn_out = alloc({1, D, hidden}, DType::F32, p + "attn_out");
        s.hidden_out = alloc({1, D, hidden}, DType::F32, p + "hidden_out");
    }
    const size_t final_norm = alloc({hidden}, DType::F32, "final_norm");
    weight_slots.push_back(final_norm);
    const size_t lm_head = alloc({hidden, vocab}, DType::BF16, "lm_head");
    weight_slots.push_back(lm_head);
    const size_t logits = alloc({1, D, vocab}, DType::F32, "logits");
    std::vector<size_t> output_slots{logits};
    output_slots.insert(output_slots.end(), present_kv.begin(), present_kv.end());

    if (weight_slots.size() != infos_.size())
        return hm_set_error(ctx_, HM_ERR_STATE, "plan expects %zu weights, model lists %zu",
                            weight_slots.size(), infos_.size());

    // attention split: rows per workgroup (kept in registers); HOMURA_ATT_CHUNK overrides
    // rows per attention split: 64 while the grid covers 2048 rows, 128 beyond (measured on 2 and 32 KV heads:
    // 1 % slower at 1024 rows, 13 % faster at 30000); HOMURA_ATT_CHUNK fixes it
    int att_chunk = 64;
    bool att_chunk_fixed = false;
    if (const char *e = std::getenv("HOMURA_ATT_CHUNK")) {
        att_chunk = std::min(128, std::max(32, std::atoi(e) / 32 * 32));
        att_chunk_fixed = true;
    }

    std::shared_ptr<PlanScratch> scr = scratch_;
    std::vector<CompiledKernel> kernels;
    std::vector<KernelStep> steps;
    auto gemv_bytes = [](double K, double N, double out_n) { return K * N * 2 + K * 4 + out_n * 4; };

    // --- Embedding kernel (reference src/hf/emitter.rs:902-909) ---
    {
        CompiledKernel k;
        k.ops_label = "Embed";
        DeviceLaunch l;
        l.name = "embed";
        l.bytes_fixed = hidden * 4.0 * 2;
        l.fn = [=](const StepContext &sc) -> int {
            Buffer *table = sc.pool[sc.step.input_slots[1]];
            Buffer *out = sc.pool[sc.step.output_slots[0]];
            return embed_step_launch(sc.ctx, sc.plan->state(), sc.plan->forced_ids(), table->as<float>(),
                                     out->as<float>(), (int)vocab, (int)hidden);
        };
        if (fused_available_) l.mode = DeviceLaunch::Mode::PerKernel;
        k.launches.push_back(std::move(l));
        if (fused_available_) {
            // One launch for the embedding row and every layer (decode_fused.hip); the layer kernels below
            // then enqueue nothing, and the last hidden state lands in the last layer's output slot.
            DeviceLaunch f;
            // ... and, unless HOMURA_WHOLE_STEP_HEAD=0, the LM head and the greedy pick as well: the step is one launch
            bool with_head = true;
            if (const char *e = std::getenv("HOMURA_WHOLE_STEP_HEAD")) with_head = std::atoi(e) != 0;
            fused_head_ = with_head;
            f.name = with_head ? "decode_whole_step[+head+pick]" : "decode_whole_step[embed+layers]";
            f.mode = DeviceLaunch::Mode::WholeStep;
            const double layer_w = (double)hidden * (qd + 2 * kvd) * 2 + (double)qd * hidden * 2 +
                                   (double)hidden * 2 * inter * 2 + (double)inter * hidden * 2;
            f.bytes_fixed = L * (layer_w + 2 * hidden * 4.0 + 2 * kvd * 2.0) + hidden * 4.0 * 2;
            if (with_head) f.bytes_fixed += gemv_bytes(hidden, vocab, vocab) + hidden * 4.0;
            f.bytes_per_kv_row = L * 2.0 * kvh * hd * 2;
            const FusedShape fs{(int)hidden, (int)H, (int)kvh, (int)hd, (int)inter};
            const size_t hidden_out_slot = ls[L - 1].hidden_out;
            const int far_only = whole_step_far_only();
            f.fn = [=](const StepContext &sc) -> int {
                FusedDecodeArgs fa{};
                fa.layers = reinterpret_cast<const FusedLayerPtrs *>(scr->fused_layers.ptr());
                fa.n_layers = L;
                fa.embed = sc.pool[sc.step.input_slots[1]]->as<float>();
                fa.vocab = (int)vocab;
                fa.state = sc.plan->state();
                fa.forced = sc.plan->forced_ids();
                fa.hidden_out = sc.pool[hidden_out_slot]->as<float>();
                fa.cos_tab = sc.pool[cos_s]->as<float>();
                fa.sin_tab = sc.pool[sin_s]->as<float>();
                fa.eps = eps;
                fa.scale = (float)(1.0 / std::sqrt((double)hd));  // f64 -> f32 constant, emitter.rs:719
                fa.max_len = sc.plan->kv_cache()->max_len();
                fa.xch = scr->fused_xch.as<unsigned char>();
                fa.ctl = scr->fused_ctl.as<uint32_t>();
                fa.trace = scr->fused_trace ? scr->fused_trace.as<unsigned long long>() : nullptr;
                fa.far_only = far_only;
                fa.spin_limit = scr->inject_spin_limit;
                fa.withhold_wg = scr->inject_withhold_wg;
                if (with_head) {
                    fa.head_w = sc.pool[lm_head]->as<uint16_t>();
                    fa.head_norm = sc.pool[final_norm]->as<float>();
                    fa.logits = sc.pool[logits]->as<float>();
                    fa.state_rw = sc.plan->state();
                    fa.out_tokens = sc.plan->out_tokens();
                    fa.out_cap = sc.plan->out_capacity();
                    fa.advance = sc.timing ? 0 : 1;
                }
                return decode_fused_launch(sc.ctx, fs, fa, sc.plan->kv_cache_len() + 1);
            };
            k.launches.push_back(std::move(f));
        }
        kernels.push_back(std::move(k));
        steps.push_back(KernelStep::kernel(kernels.size() - 1, {input_ids, embed_w}, {embed_out}));
    }

    for (int i = 0; i < L; i++) {
        const LayerSlots &s = ls[i];
        // --- QKV + QK-norm + RoPE kernel (reference src/hf/emitter.rs:915-948) ---
        {
            CompiledKernel k;
            k.ops_label = qkn ? "QKV+QKNorm+RoPE" : "QKV+RoPE";
            // The QK-norm, RoPE and cache append of this reference kernel run in the prologue of
            // the attention kernel that follows (same arithmetic, one launch fewer); the q|k|v
            // slots therefore hold the raw projections.
            DeviceLaunch g1;
            g1.name = "gemv_bf16[qkv]";
            g1.bytes_fixed = gemv_bytes(hidden, qd + 2 * kvd, qd + 2 * kvd) + hidden * 4.0;
            const size_t q_bias_slot = s.q_b;
            g1.fn = [=](const StepContext &sc) -> int {
                const auto &in = sc.step.input_slots;
                GemvArgs g;
                g.x = sc.pool[in[0]]->as<float>();
                g.w = sc.pool[in[2]]->as<uint16_t>();  // q|k|v rows are adjacent in the packed buffer
                if (q_bias_slot != (size_t)-1) g.bias = sc.pool[q_bias_slot]->as<float>();  // and so are the biases
                g.out = sc.pool[sc.step.output_slots[0]]->as<float>();  // q|k|v outputs adjacent too
                g.K = (int)hidden;
                g.N = (int)(qd + 2 * kvd);
                g.norm_w = sc.pool[in[1]]->as<float>();
                g.eps = eps;
                return gemv_bf16_nk_launch(sc.ctx, g, 1, GEMV_EPI_NONE);
            };
            if (fused_available_) g1.mode = DeviceLaunch::Mode::PerKernel;
            k.launches.push_back(std::move(g1));
            kernels.push_back(std::move(k));
            // h, ln_w, q_w, [q_b], k_w, [k_b], v_w, [v_b], cos, sin, [q_norm_w, k_norm_w]
            std::vector<size_t> in{s.hidden_in, s.input_ln, s.q_w};
            if (s.q_b != (size_t)-1) in.push_back(s.q_b);
            in.push_back(s.k_w);
            if (s.k_b != (size_t)-1) in.push_back(s.k_b);
            in.push_back(s.v_w);
            if (s.v_b != (size_t)-1) in.push_back(s.v_b);
            in.push_back(cos_s);
            in.push_back(sin_s);
            if (qkn) {
                in.push_back(s.q_norm);
                in.push_back(s.k_norm);
            }
            steps.push_back(KernelStep::kernel(kernels.size() - 1, in, {s.q, s.k, s.v}));
        }
        // --- KV concat native ops (reference src/hf/emitter.rs:950-965) ---
        for (int kv = 0; kv < 2; kv++) {
            KernelStep st;
            st.input_slots = {kv ? s.past_v : s.past_k, kv ? s.v : s.k};
            st.output_slots = {kv ? s.present_v : s.present_k};
            st.native_op = NativeOp{NativeOpKind::Concat, 2};
            steps.push_back(st);
        }
        // --- Attention + O projection kernel (reference src/hf/emitter.rs:967-980) ---
        {
            CompiledKernel k;
            k.ops_label = "Attn";
            DeviceLaunch a1;
            a1.name = qkn ? "qknorm_rope_append+gqa_attn" : "rope_append+gqa_attn";
            a1.bytes_fixed = (qd + 2 * kvd) * 4.0 + qd * 4.0 + 2 * kvd * 2.0;
            a1.bytes_per_kv_row = 2.0 * kvh * hd * 2;
            const size_t q_norm_slot = s.q_norm, k_norm_slot = s.k_norm;
            auto attn_args = [=](const StepContext &sc, int phase) {
                const auto &in = sc.step.input_slots;
                AttnArgs a;
                a.qkv_raw = sc.pool[in[0]]->as<float>();  // q|k|v raw rows are adjacent
                if (qkn) {
                    a.qw = sc.pool[q_norm_slot]->as<float>();
                    a.kw = sc.pool[k_norm_slot]->as<float>();
                }
                a.cos_tab = sc.pool[cos_s]->as<float>();
                a.sin_tab = sc.pool[sin_s]->as<float>();
                a.eps = eps;
                a.kcache = sc.pool[in[1]]->as<uint16_t>();
                a.vcache = sc.pool[in[2]]->as<uint16_t>();
                a.out = scr->attn_flat.as<float>();
                a.B = 1;
                a.H = (int)H;
                a.kvh = (int)kvh;
                a.hd = (int)hd;
                a.max_len = sc.plan->kv_cache()->max_len();
                a.kv_len = 1;
                a.scale = (float)(1.0 / std::sqrt((double)hd));  // f64 -> f32 constant, emitter.rs:719
                a.state = sc.plan->state();
                a.span = sc.plan->attn_span();
                a.fixed_chunk = att_chunk_fixed || a.span <= 2048 ? att_chunk : 128;
                a.phase = phase;
                return a;
            };
            a1.fn = [=](const StepContext &sc) -> int {
                return gqa_decode_attn_launch(sc.ctx, attn_args(sc, AttnArgs::SPLIT_ONLY));
            };
            if (fused_available_) a1.mode = DeviceLaunch::Mode::PerKernel;
            k.launches.push_back(std::move(a1));
            DeviceLaunch a1b;
            a1b.name = "gqa_attn_fold";
            a1b.bytes_fixed = qd * 4.0;
            a1b.bytes_per_kv_row = (double)(qd + 2 * H) * 4.0 / att_chunk;  // partials: one set per chunk
            a1b.fn = [=](const StepContext &sc) -> int {
                return gqa_decode_attn_launch(sc.ctx, attn_args(sc, AttnArgs::FOLD_ONLY));
            };
            a1 = std::move(a1b);
            if (fused_available_) a1.mode = DeviceLaunch::Mode::PerKernel;
            k.launches.push_back(std::move(a1));
            DeviceLaunch a2;
            a2.name = "gemv_bf16[o]";
            a2.bytes_fixed = gemv_bytes(qd, hidden, hidden);
            a2.fn = [=](const StepContext &sc) -> int {
                GemvArgs g;
                g.x = scr->attn_flat.as<float>();
                g.w = sc.pool[sc.step.input_slots[4]]->as<uint16_t>();
                g.out = sc.pool[sc.step.output_slots[0]]->as<float>();
                g.K = (int)qd;
                g.N = (int)hidden;
                return gemv_bf16_nk_launch(sc.ctx, g, 1, GEMV_EPI_NONE);
            };
            if (fused_available_) a2.mode = DeviceLaunch::Mode::PerKernel;
            k.launches.push_back(std::move(a2));
            kernels.push_back(std::move(k));
            steps.push_back(KernelStep::kernel(kernels.size() - 1,
                                               {s.q, s.present_k, s.present_v, mask, s.o_w}, {s.attn_out}));
        }
        // --- residual + MLP kernel (reference src/hf/emitter.rs:982-996) ---
        {
            CompiledKernel k;
            k.ops_label = "MLP";
            DeviceLaunch m1;
            m1.name = "gemv_bf16[gate_up+silu]";
            m1.bytes_fixed = gemv_bytes(hidden, 2 * inter, inter) + hidden * 4.0 * 3;
            m1.fn = [=](const StepContext &sc) -> int {
                const auto &in = sc.step.input_slots;
                GemvArgs g;  // gate|up interleaved rows, silu(gate)*up in the epilogue
                g.x = sc.pool[in[0]]->as<float>();
                g.prologue_residual = sc.pool[in[1]]->as<float>();
                g.norm_w = sc.pool[in[2]]->as<float>();
                g.eps = eps;
                g.resid_out = scr->resid.as<float>();
                g.w = sc.pool[in[3]]->as<uint16_t>();
                g.out = scr->act.as<float>();
                g.K = (int)hidden;
                g.N = (int)(2 * inter);
                return gemv_bf16_nk_launch(sc.ctx, g, 1, GEMV_EPI_SILU_MUL_PAIRS);
            };
            if (fused_available_) m1.mode = DeviceLaunch::Mode::PerKernel;
            k.launches.push_back(std::move(m1));
            DeviceLaunch m2;
            m2.name = "gemv_bf16[down+residual]";
            m2.bytes_fixed = gemv_bytes(inter, hidden, hidden) + hidden * 4.0;
            m2.fn = [=](const StepContext &sc) -> int {
                GemvArgs d;
                d.x = scr->act.as<float>();
                d.w = sc.pool[sc.step.input_slots[5]]->as<uint16_t>();
                d.out = sc.pool[sc.step.output_slots[0]]->as<float>();
                d.K = (int)inter;
                d.N = (int)hidden;
                d.epilogue_residual = scr->resid.as<float>();
                return gemv_bf16_nk_launch(sc.ctx, d, 1, GEMV_EPI_RESIDUAL);
            };
            if (fused_available_) m2.mode = DeviceLaunch::Mode::PerKernel;
            k.launches.push_back(std::move(m2));
            kernels.push_back(std::move(k));
            steps.push_back(KernelStep::kernel(
                kernels.size() - 1, {s.hidden_in, s.attn_out, s.post_ln, s.gate_w, s.up_w, s.down_w},
                {s.hidden_out}));
        }
    }
    // --- LM head kernel (reference src/hf/emitter.rs:999-1014) + the greedy pick of
    //     src/generate.rs:735-742 taken on the device ---
    {
        CompiledKernel k;
        k.ops_label = "LMHead";
        DeviceLaunch h1;
        h1.name = "gemv_bf16[lm_head+argmax]";
        h1.bytes_fixed = gemv_bytes(hidden, vocab, vocab) + hidden * 4.0;
        h1.fn = [=](const StepContext &sc) -> int {
            const auto &in = sc.step.input_slots;
            GemvArgs g;
            g.x = sc.pool[in[0]]->as<float>();
            g.norm_w = sc.pool[in[1]]->as<float>();
            g.eps = eps;
            g.w = sc.pool[in[2]]->as<uint16_t>();
            g.out = sc.pool[sc.step.output_slots[0]]->as<float>();
            g.K = (int)hidden;
            g.N = (int)vocab;
            g.argmax_val = scr->cand_val.as<float>();
            g.argmax_idx = scr->cand_idx.as<int>();
            g.argmax_cap = scr->cand_cap;
            return gemv_bf16_nk_launch(sc.ctx, g, 1, GEMV_EPI_ARGMAX);
        };
        if (fused_available_ && fused_head_) h1.mode = DeviceLaunch::Mode::PerKernel;
        k.launches.push_back(std::move(h1));
        DeviceLaunch h2;
        h2.name = "finish_step";
        h2.moves_cursor = true;
        h2.bytes_fixed = 64;
        if (fused_available_ && fused_head_) h2.mode = DeviceLaunch::Mode::PerKernel;
        h2.fn = [=](const StepContext &sc) -> int {
            const int ncand = std::min(gemv_bf16_nk_grid(sc.ctx, (int)vocab, 4), scr->cand_cap);
            return finish_step_launch(sc.ctx, sc.plan->state(), scr->cand_val.as<float>(),
                                      scr->cand_idx.as<int>(), ncand, sc.plan->out_tokens(),
                                      sc.plan->out_capacity());
        };
        k.launches.push_back(std::move(h2));
        kernels.push_back(std::move(k));
        steps.push_back(KernelStep::kernel(kernels.size() - 1, {ls[L - 1].hidden_out, final_norm, lm_head},
                                           {logits}));
    }

    const size_t num_slots = descs.size();
    plan_.reset(new ExecutionPlan(ctx_, std::move(kernels), std::move(steps), num_slots, input_slots,
                                  weight_slots, output_slots, std::move(descs)));
    KvPlanInfo info;
    info.num_layers = L;
    info.num_heads = (int)kvh;
    info.head_dim = (int)hd;
    info.past_kv_input_slots = past_kv;
    info.present_kv_output_slots = present_kv;
    plan_->set_kv_info(info);
    for (int i = 0; i < L; i++) {  // q|k|v of a layer share one allocation
        plan_->alias_slot(ls[i].k, ls[i].q, (size_t)qd * 4);
        plan_->alias_slot(ls[i].v, ls[i].q, (size_t)(qd + kvd) * 4);
    }
    return HM_OK;
}

// ── quantised plan ───────────────────────────────────────────────────────────
// Step list of emit_transformer_plan_quant (reference src/hf/emitter_quant.rs:1211-1440), one
// KernelStep per reference step: RMSNorm, QuantMM Q/K/V, PostQKV, KV concat x2, AttnBody,
// QuantMM O, Residual+Norm, QuantMM Gate/Up, SiLU*Up, QuantMM Down, ResAdd; f32 LM head.
// Fusions that keep the arithmetic: the Q step's launch covers K and V too (their blocks are
// stored back to back), Gate's covers Up, and PostQKV runs in AttnBody's prologue. The
// reference's f64 accumulations (sum of squares, sum of exps) are f32 tree sums here.
int HfModel::emit_transformer_plan_quant() {
    const TransformerConfig c = cfg_;
    const int64_t hidden = c.hidden_size, inter = c.intermediate_size, vocab = c.vocab_size;
    const int64_t H = c.num_attention_heads, kvh = c.kv_heads(), hd = c.head_dim();
    const int64_t qd = c.q_dim(), kvd = c.kv_dim();
    const int L = c.num_hidden_layers;
    const float eps = (float)c.rms_norm_eps;
    const bool qkn = has_qk_norm_;
    const int64_t D = DIM_DYNAMIC;

    std::vector<SlotDesc> descs;
    auto alloc = [&](std::vector<int64_t> shape, DType dt, const std::string &name) -> size_t {
        descs.push_back(SlotDesc{std::move(shape), dt, name});
        return descs.size() - 1;
    };
    std::vector<size_t> input_slots, weight_slots, past_kv, present_kv;
    const size_t input_ids = alloc({1, D}, DType::I64, "input_ids");
    const size_t mask = alloc({1, 1, D, D}, DType::F32, "mask");
    const size_t cos_s = alloc({D, hd}, DType::F32, "cos");
    const size_t sin_s = alloc({D, hd}, DType::F32, "sin");
    input_slots = {input_ids, mask, cos_s, sin_s};
    const size_t embed_w = alloc({vocab, hidden}, DType::F32, "embed_tokens");
    weight_slots.push_back(embed_w);
    const size_t embed_out = alloc({1, D, hidden}, DType::F32, "embed_out");

    struct LS {
        size_t hidden_in, input_ln, q_w, k_w, v_w, q_b, k_b, v_b, q_norm, k_norm, o_w, post_ln, gate_w, up_w, down_w;
        size_t past_k, past_v, present_k, present_v;
        size_t normed, q_out, k_out, v_out, q, k_bhsd, v_bhsd, attn_body, attn_out, residual, post_normed,
            gate_out, up_out, silu, down_out, hidden_out;
    };
    std::vector<LS> ls(L);
    auto qbytes = [&](DType t, int64_t K, int64_t N) {
        return (int64_t)dtype_bytes_for_elements(t, (size_t)(K * N), nullptr);
    };
    for (int i = 0; i < L; i++) {
        LS &s = ls[i];
        const std::string p = "l" + std::to_string(i) + ".";
        s.hidden_in = i == 0 ? embed_out : ls[i - 1].hidden_out;
        auto w = [&](std::vector<int64_t> shape, DType dt, const std::string &n) {
            size_t slot = alloc(std::move(shape), dt, p + n);
            weight_slots.push_back(slot);
            return slot;
        };
        // quantised weights are flat byte buffers (reference src/hf/emitter_quant.rs:213-222)
        s.input_ln = w({hidden}, DType::F32, "input_ln");
        const bool bias = c.attention_bias;
        s.q_b = s.k_b = s.v_b = (size_t)-1;
        const DType tq = proj_dtype(i, 0), tk = proj_dtype(i, 1), tv = proj_dtype(i, 2), to = proj_dtype(i, 3),
                    tg = proj_dtype(i, 4), tu = proj_dtype(i, 5), td = proj_dtype(i, 6);
        s.q_w = w({qbytes(tq, hidden, qd)}, tq, "q_w");
        if (bias) s.q_b = w({qd}, DType::F32, "q_b");
        s.k_w = w({qbytes(tk, hidden, kvd)}, tk, "k_w");
        if (bias) s.k_b = w({kvd}, DType::F32, "k_b");
        s.v_w = w({qbytes(tv, hidden, kvd)}, tv, "v_w");
        if (bias) s.v_b = w({kvd}, DType::F32, "v_b");
        s.q_norm = s.k_norm = (size_t)-1;
        if (qkn) {
            s.q_norm = w({hd}, DType::F32, "q_norm");
            s.k_norm = w({hd}, DType::F32, "k_norm");
        }
        s.o_w = w({qbytes(to, qd, hidden)}, to, "o_w");
        s.post_ln = w({hidden}, DType::F32, "post_ln");
        s.gate_w = w({qbytes(tg, hidden, inter)}, tg, "gate_w");
        s.up_w = w({qbytes(tu, hidden, inter)}, tu, "up_w");
        s.down_w = w({qbytes(td, inter, hidden)}, td, "down_w");
        s.past_k = alloc({1, kvh, D, hd}, DType::BF16, p + "past_k");
        s.past_v = alloc({1, kvh, D, hd}, DType::BF16, p + "past_v");
        past_kv.push_back(s.past_k);
        past_kv.push_back(s.past_v);
        input_slots.push_back(s.past_k);
        input_slots.push_back(s.past_v);
        s.present_k = alloc({1, kvh, D, hd}, DType::BF16, p + "present_k");
        s.present_v = alloc({1, kvh, D, hd}, DType::BF16, p + "present_v");
        present_kv.push_back(s.present_k);
        present_kv.push_back(s.present_v);
        s.normed = alloc({1, D, hidden}, DType::F32, p + "normed");
        s.q_out = alloc({1, D, qd}, DType::F32, p + "q_proj_out");
        s.k_out = alloc({1, D, kvd}, DType::F32, p + "k_proj_out");
        s.v_out = alloc({1, D, kvd}, DType::F32, p + "v_proj_out");
        s.q = alloc({1, D, H, hd}, DType::F32, p + "q");
        s.k_bhsd = alloc({1, kvh, D, hd}, DType::F32, p + "k_bhsd");
        s.v_bhsd = alloc({1, kvh, D, hd}, DType::F32, p + "v_bhsd");
        s.attn_body = alloc({1, D, qd}, DType::F32, p + "attn_body_out");
        s.attn_out = alloc({1, D, hidden}, DType::F32, p + "attn_out");
        s.residual = alloc({1, D, hidden}, DType::F32, p + "residual");
        s.post_normed = alloc({1, D, hidden}, DType::F32, p + "post_attn_normed");
        s.gate_out = alloc({1, D, inter}, DType::F32, p + "gate_out");
        s.up_out = alloc({1, D, inter}, DType::F32, p + "up_out");
        s.silu = alloc({1, D, inter}, DType::F32, p + "silu_mul_out");
        s.down_out = alloc({1, D, hidden}, DType::F32, p + "down_out");
        s.hidden_out = alloc({1, D, hidden}, DType::F32, p + "hidden_out");
    }
    const size_t final_norm = alloc({hidden}, DType::F32, "final_norm");
    weight_slots.push_back(final_norm);
    const size_t lm_head = alloc({hidden, vocab}, DType::F32, "lm_head");
    weight_slots.push_back(lm_head);
    const size_t logits = alloc({1, D, vocab}, DType::F32, "logits");
    std::vector<size_t> output_slots{logits};
    output_slots.insert(output_slots.end(), present_kv.begin(), present_kv.end());
    if (weight_slots.size() != infos_.size())
        return hm_set_error(ctx_, HM_ERR_STATE, "plan expects %zu weights, model lists %zu",
                            weight_slots.size(), infos_.size());

    // rows per attention split: 64 while the grid covers 2048 rows, 128 beyond (measured on 2 and 32 KV heads:
    // 1 % slower at 1024 rows, 13 % faster at 30000); HOMURA_ATT_CHUNK fixes it
    int att_chunk = 64;
    bool att_chunk_fixed = false;
    if (const char *e = std::getenv("HOMURA_ATT_CHUNK")) {
        att_chunk = std::min(128, std::max(32, std::atoi(e) / 32 * 32));
        att_chunk_fixed = true;
    }

    std::shared_ptr<PlanScratch> scr = scratch_;
    std::vector<CompiledKernel> kernels;
    std::vector<KernelStep> steps;
    auto add_step = [&](CompiledKernel k, std::vector<size_t> in, std::vector<size_t> out) {
        kernels.push_back(std::move(k));
        steps.push_back(KernelStep::kernel(kernels.size() - 1, std::move(in), std::move(out)));
    };
    // QuantMM step (reference emit_quant_matmul_kernel, src/hf/emitter_quant.rs:675-702): inputs
    // [activation, weight bytes], output [1, seq, N]. The first matrix of a stacked run launches over
    // the whole run (N rows = the run's total, its outputs are adjacent too); the others launch
    // nothing. reuse_act: an earlier K-quant launch of the same group already quantised this
    // activation.
    // Light ops of the neighbouring steps that a Q8_0 / Q4_0 launch does on its way (slots; NO = none):
    // x <- silu(x) * x2 | x <- x + res_in (-> resid_out) | x <- rmsnorm(x) * norm_w | out <- dot + add.
    // x / out replace the step's own activation and output slot.
    constexpr size_t NO = (size_t)-1;
    struct FuseSlots { size_t x = (size_t)-1, x2 = (size_t)-1, res_in = (size_t)-1, resid_out = (size_t)-1,
                              norm_w = (size_t)-1, add = (size_t)-1, out = (size_t)-1;
                       bool silu_pairs = false; };
    // A second run of the group that rides in the first run's launch (the two K-quant types side by side)
    struct PairedRun { size_t w_slot = (size_t)-1, out_slot = (size_t)-1; int64_t N = 0; DType dtype = DType::F32; std::string label; };
    auto quant_mm = [&](const char *label, DType wdt, int64_t K, int64_t N, bool reuse_act, FuseSlots fs,
                        PairedRun pair = PairedRun(), const uint8_t *planes = nullptr) {
        CompiledKernel k;
        k.ops_label = std::string("QuantMM[") + label + "]";
        if (N > 0 && pair.N > 0) {
            DeviceLaunch l;
            l.name = std::string(wdt == DType::Q4_K ? "gemv_q4_k+q6_k[" : "gemv_q6_k+q4_k[") + label + "|" + pair.label + "]";
            if (fs.norm_w != NO) l.name += fs.res_in != NO ? "+resid+norm" : "+norm";
            l.bytes_fixed = (double)dtype_bytes_for_elements(wdt, (size_t)(K * N), nullptr) +
                            (double)dtype_bytes_for_elements(pair.dtype, (size_t)(K * pair.N), nullptr) + K * 4.0 + (N + pair.N) * 4.0;
            l.fn = [=](const StepContext &sc) -> int {
                auto f32 = [&](size_t slot) { return slot == NO ? nullptr : sc.pool[slot]->as<float>(); };
                const float *x = fs.x != NO ? f32(fs.x) : sc.pool[sc.step.input_slots[0]]->as<float>();
                float *out = fs.out != NO ? f32(fs.out) : sc.pool[sc.step.output_slots[0]]->as<float>();
                QuantFuse f;
                f.res_in = f32(fs.res_in);
                f.resid_out = f32(fs.resid_out);
                f.norm_w = f32(fs.norm_w);
                f.eps = eps;
                return gemv_kquant_fused_pair(sc.ctx, wdt == DType::Q6_K, x, sc.pool[sc.step.input_slots[1]]->as<uint8_t>(), out, (int)N,
                                              sc.pool[pair.w_slot]->as<uint8_t>(), sc.pool[pair.out_slot]->as<float>(), (int)pair.N,
                                              (int)K, f);
            };
            k.launches.push_back(std::move(l));
        } else if (N > 0) {
            DeviceLaunch l;
            const char *kn = wdt == DType::Q8_0 ? "gemv_q8_0[" : wdt == DType::Q4_0 ? "gemv_q4_0["
                             : wdt == DType::Q4_K ? "gemv_q4_k[" : "gemv_q6_k[";
            l.name = std::string(kn) + label + "]";
            if (fs.norm_w != NO) l.name += fs.res_in != NO ? "+resid+norm" : "+norm";
            if (fs.x2 != NO) l.name += "+silu";
            if (fs.add != NO) l.name += "+resid";
            l.bytes_fixed = (double)dtype_bytes_for_elements(wdt, (size_t)(K * N), nullptr) + K * 4.0 + N * 4.0;
            l.fn = [=](const StepContext &sc) -> int {
                auto f32 = [&](size_t slot) { return slot == NO ? nullptr : sc.pool[slot]->as<float>(); };
                const float *x = fs.x != NO ? f32(fs.x) : sc.pool[sc.step.input_slots[0]]->as<float>();
                const uint8_t *w = sc.pool[sc.step.input_slots[1]]->as<uint8_t>();
                float *out = fs.out != NO ? f32(fs.out) : sc.pool[sc.step.output_slots[0]]->as<float>();
                QuantFuse f;
                f.x2 = f32(fs.x2);
                f.res_in = f32(fs.res_in);
                f.resid_out = f32(fs.resid_out);
                f.norm_w = f32(fs.norm_w);
                f.eps = eps;
                f.res_out_add = f32(fs.add);
                if (planes)  // the run re-packed at finalize
                    return gemv_planes_fused(sc.ctx, wdt == DType::Q4_0, x, planes, out, (int)K, (int)N, f);
                if (wdt == DType::Q8_0 || wdt == DType::Q4_0)
                    return gemv_quant_fused(sc.ctx, wdt == DType::Q4_0, x, w, out, (int)K, (int)N, f);
                if (K <= 4096)  // the row is prepared and quantised to Q8_K inside the kernel
                    return gemv_kquant_fused(sc.ctx, wdt == DType::Q6_K, x, w, out, (int)K, (int)N, f);
                return gemv_kquant(sc.ctx, wdt == DType::Q6_K, x, w, out, (int)K, (int)N, reuse_act);
            };
            k.launches.push_back(std::move(l));
        }
        return k;
    };
    // Whether every launch of a group can take light ops along: Q8_0 / Q4_0 always, K-quants while the
    // row fits the in-kernel preparation
    auto plain_group = [&](int layer, std::initializer_list<int> which, int64_t K) {
        if (packed_[layer].k8[0]) return true;  // the K8 launch prepares rows of any width it serves
        for (int w : which) {
            const DType t = proj_dtype(layer, w);
            if ((t == DType::Q4_K || t == DType::Q6_K) && K > 4096) return false;
        }
        return true;
    };
    // The QuantMM steps of one group of matrices that share an activation (q|k|v, gate|up, or one alone)
    struct GroupMember { const char *label; int which; int64_t N; size_t w_slot, out_slot; };
    auto quant_group = [&](int layer, size_t act_slot, int64_t K, std::vector<GroupMember> members, FuseSlots fs) {
        // A model whose K-quant matrices were re-packed into the K8 form: one launch for the whole group, whatever
        // mix of Q4_K and Q6_K its members are (their outputs are adjacent); the row is prepared and quantised to
        // Q8_K inside the launch. The step list keeps the reference's kernels; the other members launch nothing.
        const int group_of[7] = {0, 0, 0, 1, 2, 2, 3};
        const Buffer &k8 = packed_[layer].k8[group_of[members[0].which]];
        if (k8 && (fs.norm_w == NO || K <= 8192)) {
            int64_t n_all = 0;
            std::string label;
            for (const GroupMember &gm : members) {
                n_all += gm.N;
                label += gm.label;
            }
            const uint8_t *plane = k8.as<uint8_t>();
            const uint8_t *records = plane + k8_plane_bytes((int)n_all, (int)K);
            for (size_t j = 0; j < members.size(); j++) {
                CompiledKernel k;
                k.ops_label = std::string("QuantMM[") + members[j].label + "]";
                if (j == 0) {
                    DeviceLaunch l;
                    l.name = "gemv_k8[" + label + "]";
                    if (fs.norm_w != NO) l.name += fs.res_in != NO ? "+resid+norm" : "+norm";
                    if (fs.x2 != NO) l.name += "+silu";
                    if (fs.silu_pairs) l.name += "+silu*up";
                    if (fs.add != NO) l.name += "+resid";
                    l.bytes_fixed = (double)k8.bytes() + K * 4.0 + n_all * 4.0;
                    const int64_t Kc = K, Nc = n_all;
                    l.fn = [=](const StepContext &sc) -> int {
                        auto f32 = [&](size_t slot) { return slot == NO ? nullptr : sc.pool[slot]->as<float>(); };
                        const float *x = fs.x != NO ? f32(fs.x) : sc.pool[sc.step.input_slots[0]]->as<float>();
                        float *out = fs.out != NO ? f32(fs.out) : sc.pool[sc.step.output_slots[0]]->as<float>();
                        QuantFuse f;
                        f.x2 = f32(fs.x2);
                        f.res_in = f32(fs.res_in);
                        f.resid_out = f32(fs.resid_out);
                        f.norm_w = f32(fs.norm_w);
                        f.eps = eps;
                        f.res_out_add = f32(fs.add);
                        f.silu_pairs = fs.silu_pairs;
                        return gemv_k8_fused(sc.ctx, x, plane, records, out, (int)Kc, (int)Nc, f);
                    };
                    k.launches.push_back(std::move(l));
                }
                add_step(std::move(k), {act_slot, members[j].w_slot}, {members[j].out_slot});
            }
            return;
        }
        // the runs of same-type neighbours: (first member, count, rows, label)
        struct Run { size_t j; int count; int64_t n; std::string label; DType t; };
        std::vector<Run> runs;
        for (size_t j = 0; j < members.size(); j++) {
            int first, count;
            quant_run(layer, members[j].which, &first, &count);
            if (first != members[j].which) continue;
            Run r{j, count, 0, "", proj_dtype(layer, members[j].which)};
            for (int e = 0; e < count; e++) {
                r.n += members[j + e].N;
                r.label += members[j + e].label;
            }
            runs.push_back(std::move(r));
        }
        auto is_k = [](DType t) { return t == DType::Q4_K || t == DType::Q6_K; };
        // two runs, one of each K-quant type, prepared in the kernel: one launch for both
        const bool paired = runs.size() == 2 && is_k(runs[0].t) && is_k(runs[1].t) && runs[0].t != runs[1].t && K <= 4096 &&
                            fs.x2 == NO && fs.add == NO && fs.out == NO;
        bool act_quantized = false;
        for (size_t j = 0; j < members.size(); j++) {
            const GroupMember &gm = members[j];
            const DType t = proj_dtype(layer, gm.which);
            const bool kq = is_k(t);
            const Run *run = nullptr;
            for (const Run &r : runs)
                if (r.j == j) run = &r;
            int64_t n_run = run ? run->n : 0;
            const std::string label = run ? run->label : std::string(gm.label);
            PairedRun pair;
            if (paired && run == &runs[0]) {
                const GroupMember &second = members[runs[1].j];
                pair.w_slot = second.w_slot;
                pair.out_slot = second.out_slot;
                pair.N = runs[1].n;
                pair.dtype = runs[1].t;
                pair.label = runs[1].label;
            } else if (paired && run == &runs[1]) {
                n_run = 0;  // rides in the first run's launch
            }
            const Buffer &pl = packed_[layer].planes[gm.which];  // set for the first member of a re-packed run
            add_step(quant_mm(label.c_str(), t, K, n_run, kq && act_quantized, fs, pair, n_run > 0 && pl ? pl.as<uint8_t>() : nullptr),
                     {act_slot, gm.w_slot}, {gm.out_slot});
            if (n_run > 0 && kq) act_quantized = true;
        }
    };

    {
        CompiledKernel k;
        k.ops_label = "Embed";
        DeviceLaunch l;
        l.name = "embed";
        l.bytes_fixed = hidden * 4.0 * 2;
        l.fn = [=](const StepContext &sc) -> int {
            return embed_step_launch(sc.ctx, sc.plan->state(), sc.plan->forced_ids(),
                                     sc.pool[sc.step.input_slots[1]]->as<float>(),
                                     sc.pool[sc.step.output_slots[0]]->as<float>(), (int)vocab, (int)hidden);
        };
        if (fused_available_) l.mode = DeviceLaunch::Mode::PerKernel;
        k.launches.push_back(std::move(l));
        if (fused_available_) {
            // One launch for the embedding row and every layer (decode_fused.hip, reading the re-packed
            // planes); the layer kernels below then enqueue nothing, and the last hidden state lands in the
            // last layer's output slot.
            DeviceLaunch f;
            f.name = "decode_whole_step[embed+layers]";
            f.mode = DeviceLaunch::Mode::WholeStep;
            double layer_w = 0;
            {
                const int64_t kd[7] = {hidden, hidden, hidden, qd, hidden, hidden, inter};
                const int64_t nd[7] = {qd, kvd, kvd, hidden, inter, inter, hidden};
                for (int j = 0; j < 7; j++) layer_w += (double)dtype_bytes_for_elements(proj_dtype(0, j), (size_t)(kd[j] * nd[j]), nullptr);
            }
            f.bytes_fixed = L * (layer_w + 2 * hidden * 4.0 + 2 * kvd * 2.0) + hidden * 4.0 * 2;
            f.bytes_per_kv_row = L * 2.0 * kvh * hd * 2;
            const FusedShape fshape{(int)hidden, (int)H, (int)kvh, (int)hd, (int)inter, fused_wf_};
            const size_t hidden_out_slot = ls[L - 1].hidden_out;
            const size_t cos_slot = cos_s, sin_slot = sin_s;
            const int far_only = whole_step_far_only();
            f.fn = [=](const StepContext &sc) -> int {
                FusedDecodeArgs fa{};
                fa.layers = reinterpret_cast<const FusedLayerPtrs *>(scr->fused_layers.ptr());
                fa.n_layers = (int)L;
                fa.embed = sc.pool[sc.step.input_slots[1]]->as<float>();
                fa.vocab = (int)vocab;
                fa.state = sc.plan->state();
                fa.forced = sc.plan->forced_ids();
                fa.hidden_out = sc.pool[hidden_out_slot]->as<float>();
                fa.cos_tab = sc.pool[cos_slot]->as<float>();
                fa.sin_tab = sc.pool[sin_slot]->as<float>();
                fa.eps = eps;
                fa.scale = (float)(1.0 / std::sqrt((double)hd));
                fa.max_len = sc.plan->kv_cache()->max_len();
                fa.xch = scr->fused_xch.as<unsigned char>();
                fa.ctl = scr->fused_ctl.as<uint32_t>();
                fa.trace = scr->fused_trace ? scr->fused_trace.as<unsigned long long>() : nullptr;
                fa.far_only = far_only;
                fa.spin_limit = scr->inject_spin_limit;
                fa.withhold_wg = scr->inject_withhold_wg;
                return decode_fused_launch(sc.ctx, fshape, fa, sc.plan->kv_cache_len() + 1);
            };
            k.launches.push_back(std::move(f));
        }
        add_step(std::move(k), {input_ids, embed_w}, {embed_out});
    }
    const size_t first_layer_kernel = kernels.size();
    for (int i = 0; i < L; i++) {
        const LS &s = ls[i];
        // Which light steps ride along with a Q8_0 / Q4_0 product instead of being launched (the step
        // list keeps the reference's kernels; a step whose work moved has no launch of its own)
        const bool fuse_in_norm = plain_group(i, {0, 1, 2}, hidden) && hidden <= 4096;
        const bool fuse_post_norm = plain_group(i, {4, 5}, hidden) && hidden <= 4096;
        const bool fuse_down = plain_group(i, {6}, inter);
        // Long Q8_0 / Q4_0 rows go through the cut-row kernel, where every workgroup would redo SiLU * up over
        // the whole row (8960 -> 1536: 12.6 us against 7.3 + a 2.5 us launch of its own; no gain below 8192)
        const bool silu_apart = fuse_down && !packed_[i].k8[3] && inter >= 8192 &&
                                (proj_dtype(i, 6) == DType::Q8_0 || proj_dtype(i, 6) == DType::Q4_0);
        {  // Step 1: pre-QKV RMSNorm (reference :713-791)
            CompiledKernel k;
            k.ops_label = "RMSNorm";
            if (!fuse_in_norm) {
                DeviceLaunch l;
                l.name = "rmsnorm";
                l.bytes_fixed = hidden * 4.0 * 3;
                l.fn = [=](const StepContext &sc) -> int {
                    return rmsnorm_launch(sc.ctx, sc.pool[sc.step.input_slots[0]]->as<float>(), nullptr,
                                          sc.pool[sc.step.input_slots[1]]->as<float>(),
                                          sc.pool[sc.step.output_slots[0]]->as<float>(), nullptr, 1, (int)hidden, eps);
                };
                k.launches.push_back(std::move(l));
            }
            add_step(std::move(k), {s.hidden_in, s.input_ln}, {s.normed});
        }
        // Steps 2-4: QuantMM Q, K, V — one launch over the stacked q|k|v rows
        // Where q|k|v multiply in one launch, the bias add of the next reference kernel rides out with it (the
        // biases are adjacent like the rows): out = dot + bias, the same single addition.
        bool bias_folded = false;
        {
            FuseSlots fs;
            if (fuse_in_norm) {
                fs.x = s.hidden_in;
                fs.norm_w = s.input_ln;
            }
            int first_run, count_run;
            quant_run(i, 0, &first_run, &count_run);
            if (s.q_b != (size_t)-1 && (packed_[i].k8[0] || count_run == 3)) {
                fs.add = s.q_b;
                bias_folded = true;
            }
            quant_group(i, s.normed, hidden, {{"q", 0, qd, s.q_w, s.q_out}, {"k", 1, kvd, s.k_w, s.k_out},
                                              {"v", 2, kvd, s.v_w, s.v_out}}, fs);
        }
        {  // Step 5: PostQKV (reference :802-912) — runs in the attention kernel's prologue
            CompiledKernel k;
            k.ops_label = qkn ? "PostQKV+QKNorm+RoPE" : "PostQKV+RoPE";
            std::vector<size_t> in{s.q_out, s.k_out, s.v_out, cos_s, sin_s};
            if (s.q_b != (size_t)-1) {
                in.push_back(s.q_b);
                in.push_back(s.k_b);
                in.push_back(s.v_b);
            }
            if (s.q_b != (size_t)-1 && !bias_folded) {
                // the bias add of this reference kernel (src/hf/emitter_quant.rs:836-850): one launch
                // over the adjacent q|k|v rows and the adjacent biases
                DeviceLaunch l;
                l.name = "qkv_bias_add";
                l.bytes_fixed = (qd + 2 * kvd) * 4.0 * 3;
                const size_t raw = s.q_out, qb = s.q_b;
                l.fn = [=](const StepContext &sc) -> int {
                    float *x = sc.pool[raw]->as<float>();
                    return hm_add(sc.ctx, x, sc.pool[qb]->as<float>(), x, (size_t)(qd + 2 * kvd));
                };
                k.launches.push_back(std::move(l));
            }
            if (qkn) {
                in.push_back(s.q_norm);
                in.push_back(s.k_norm);
            }
            add_step(std::move(k), in, {s.q, s.k_bhsd, s.v_bhsd});
        }
        for (int kv = 0; kv < 2; kv++) {  // Steps 6-7: KV concat
            KernelStep st;
            st.input_slots = {kv ? s.past_v : s.past_k, kv ? s.v_bhsd : s.k_bhsd};
            st.output_slots = {kv ? s.present_v : s.present_k};
            st.native_op = NativeOp{NativeOpKind::Concat, 2};
            steps.push_back(st);
        }
        {  // Step 8: AttnBody (reference :922-975)
            CompiledKernel k;
            k.ops_label = "AttnBody";
            DeviceLaunch l;
            l.name = qkn ? "qknorm_rope_append+gqa_attn" : "rope_append+gqa_attn";
            l.bytes_fixed = (qd + 2 * kvd) * 4.0 + qd * 4.0 + 2 * kvd * 2.0;
            l.bytes_per_kv_row = 2.0 * kvh * hd * 2;
            const size_t raw_slot = s.q_out, qn = s.q_norm, kn = s.k_norm;
            auto attn_args = [=](const StepContext &sc, int phase) {
                const auto &in = sc.step.input_slots;
                AttnArgs a;
                a.qkv_raw = sc.pool[raw_slot]->as<float>();
                if (qkn) {
                    a.qw = sc.pool[qn]->as<float>();
                    a.kw = sc.pool[kn]->as<float>();
                }
                a.cos_tab = sc.pool[cos_s]->as<float>();
                a.sin_tab = sc.pool[sin_s]->as<float>();
                a.eps = eps;
                a.kcache = sc.pool[in[1]]->as<uint16_t>();
                a.vcache = sc.pool[in[2]]->as<uint16_t>();
                a.out = sc.pool[sc.step.output_slots[0]]->as<float>();
                a.B = 1;
                a.H = (int)H;
                a.kvh = (int)kvh;
                a.hd = (int)hd;
                a.max_len = sc.plan->kv_cache()->max_len();
                a.kv_len = 1;
                a.scale = (float)(1.0 / std::sqrt((double)hd));
                a.state = sc.plan->state();
                a.span = sc.plan->attn_span();
                a.fixed_chunk = att_chunk_fixed || a.span <= 2048 ? att_chunk : 128;
                a.phase = phase;
                return a;
            };
            l.fn = [=](const StepContext &sc) -> int {
                return gqa_decode_attn_launch(sc.ctx, attn_args(sc, AttnArgs::SPLIT_ONLY));
            };
            k.launches.push_back(std::move(l));
            DeviceLaunch lf;
            lf.name = "gqa_attn_fold";
            lf.bytes_fixed = qd * 4.0;
            lf.bytes_per_kv_row = (double)(qd + 2 * H) * 4.0 / att_chunk;
            lf.fn = [=](const StepContext &sc) -> int {
                return gqa_decode_attn_launch(sc.ctx, attn_args(sc, AttnArgs::FOLD_ONLY));
            };
            l = std::move(lf);
            k.launches.push_back(std::move(l));
            add_step(std::move(k), {s.q, s.present_k, s.present_v, mask}, {s.attn_body});
        }
        quant_group(i, s.attn_body, qd, {{"o", 3, hidden, s.o_w, s.attn_out}}, FuseSlots());  // Step 9
        {  // Step 10: Residual + RMSNorm (reference :985-1071), two outputs
            CompiledKernel k;
            k.ops_label = "Residual+Norm";
            if (!fuse_post_norm) {
                DeviceLaunch l;
                l.name = "residual_rmsnorm";
                l.bytes_fixed = hidden * 4.0 * 5;
                l.fn = [=](const StepContext &sc) -> int {
                    const auto &in = sc.step.input_slots;
                    return rmsnorm_launch(sc.ctx, sc.pool[in[0]]->as<float>(), sc.pool[in[1]]->as<float>(),
                                          sc.pool[in[2]]->as<float>(), sc.pool[sc.step.output_slots[1]]->as<float>(),
                                          sc.pool[sc.step.output_slots[0]]->as<float>(), 1, (int)hidden, eps);
                };
                k.launches.push_back(std::move(l));
            }
            add_step(std::move(k), {s.hidden_in, s.attn_out, s.post_ln}, {s.residual, s.post_normed});
        }
        {  // Steps 11-12: QuantMM Gate, Up — one launch per run of equal types over the stacked rows
            FuseSlots fs;
            if (fuse_post_norm) {  // residual = hidden_in + attn_out, normed on the way in
                fs.x = s.hidden_in;
                fs.res_in = s.attn_out;
                fs.resid_out = s.residual;
                fs.norm_w = s.post_ln;
            }
            if (k8_pairs_ && packed_[i].k8[2]) {  // interleaved rows: SiLU * up leaves this launch (Step 13's work)
                fs.silu_pairs = true;
                fs.out = s.silu;
            }
            quant_group(i, s.post_normed, hidden, {{"gate", 4, inter, s.gate_w, s.gate_out}, {"up", 5, inter, s.up_w, s.up_out}}, fs);
        }
        {  // Step 13: SiLU * Up (reference :1077-1103)
            CompiledKernel k;
            k.ops_label = "SiLU*Up";
            if (!fuse_down || silu_apart) {
                DeviceLaunch l;
                l.name = "silu_mul";
                l.bytes_fixed = inter * 4.0 * 3;
                l.fn = [=](const StepContext &sc) -> int {
                    const auto &in = sc.step.input_slots;
                    return hm_silu_mul(sc.ctx, sc.pool[in[0]]->as<float>(), sc.pool[in[1]]->as<float>(),
                                       sc.pool[sc.step.output_slots[0]]->as<float>(), (size_t)inter);
                };
                k.launches.push_back(std::move(l));
            }
            add_step(std::move(k), {s.gate_out, s.up_out}, {s.silu});
        }
        {  // Step 14: QuantMM Down; with a Q8_0 / Q4_0 matrix it takes SiLU*Up on the way in and ResAdd on the way out
            FuseSlots fs;
            if (fuse_down) {
                if (!(k8_pairs_ && packed_[i].k8[2]) && !silu_apart) {  // else SiLU * up already sits in the step's own input
                    fs.x = s.gate_out;
                    fs.x2 = s.up_out;
                }
                fs.add = s.residual;
                fs.out = s.hidden_out;
            }
            quant_group(i, s.silu, inter, {{"down", 6, hidden, s.down_w, s.down_out}}, fs);
        }
        {  // Step 15: ResAdd (reference :1109-1134)
            CompiledKernel k;
            k.ops_label = "ResAdd";
            if (!fuse_down) {
                DeviceLaunch l;
                l.name = "residual_add";
                l.bytes_fixed = hidden * 4.0 * 3;
                l.fn = [=](const StepContext &sc) -> int {
                    const auto &in = sc.step.input_slots;
                    return hm_add(sc.ctx, sc.pool[in[0]]->as<float>(), sc.pool[in[1]]->as<float>(),
                                  sc.pool[sc.step.output_slots[0]]->as<float>(), (size_t)hidden);
                };
                k.launches.push_back(std::move(l));
            }
            add_step(std::move(k), {s.residual, s.down_out}, {s.hidden_out});
        }
    }
    if (fused_available_)  // in whole-step mode the layers' own launches stay out
        for (size_t ki = first_layer_kernel; ki < kernels.size(); ki++)
            for (DeviceLaunch &dl : kernels[ki].launches) dl.mode = DeviceLaunch::Mode::PerKernel;
    {  // LM head: final RMSNorm + f32 matmul (reference :1399-1440) + device-side greedy pick
        CompiledKernel k;
        k.ops_label = "LMHead";
        DeviceLaunch h1;
        const bool head_blocks = (bool)lm_head_blocks_;
        const DType head_dt = lm_head_blocks_dtype_;
        const bool head_q6 = head_dt == DType::Q6_K;
        const bool head_k = head_dt == DType::Q4_K || head_dt == DType::Q6_K;  // else Q8_0 / Q4_0
        const uint8_t *head_planes = lm_head_planes_ ? lm_head_planes_.as<uint8_t>() : nullptr;
        h1.name = !head_blocks ? "gemv_f32[lm_head+argmax]"
                  : head_q6    ? "gemv_q6_k_f32[lm_head+argmax]"
                  : head_k     ? "gemv_q4_k_f32[lm_head+argmax]"
                  : head_dt == DType::Q8_0 ? "gemv_q8_0[lm_head+argmax]" : "gemv_q4_0[lm_head+argmax]";
        h1.bytes_fixed = (head_blocks ? (double)lm_head_blocks_.bytes() : (double)hidden * vocab * 4) + hidden * 8.0 + vocab * 4.0;
        h1.fn = [=](const StepContext &sc) -> int {
            const auto &in = sc.step.input_slots;
            if (head_blocks && !head_k) {  // Q8_0 / Q4_0: the dequant-GEMV of the projections, norm in, candidates out
                QuantFuse f;
                f.norm_w = sc.pool[in[1]]->as<float>();
                f.eps = eps;
                f.cand_v = scr->cand_val.as<float>();
                f.cand_i = scr->cand_idx.as<int>();
                if (head_planes)
                    return gemv_planes_fused(sc.ctx, head_dt == DType::Q4_0, sc.pool[in[0]]->as<float>(), head_planes,
                                             sc.pool[sc.step.output_slots[0]]->as<float>(), (int)hidden, (int)vocab, f);
                return gemv_quant_fused(sc.ctx, head_dt == DType::Q4_0, sc.pool[in[0]]->as<float>(), sc.pool[in[2]]->as<uint8_t>(),
                                        sc.pool[sc.step.output_slots[0]]->as<float>(), (int)hidden, (int)vocab, f);
            }
            if (head_q6 && head_planes)  // the same product over the re-packed output matrix
                return gemv_q6k_planes_f32(sc.ctx, "gemv_q6_k_f32_planes[head]", sc.pool[in[0]]->as<float>(), sc.pool[in[1]]->as<float>(), eps,
                                           head_planes, sc.pool[sc.step.output_slots[0]]->as<float>(), 1, (int)hidden, (int)vocab,
                                           scr->cand_val.as<float>(), scr->cand_idx.as<int>(), scr->cand_cap);
            if (head_blocks)  // the f32 product with the dequantised output matrix, read from its blocks
                return gemv_kquant_f32_head(sc.ctx, head_q6, sc.pool[in[0]]->as<float>(), sc.pool[in[1]]->as<float>(), eps,
                                            sc.pool[in[2]]->as<uint8_t>(), sc.pool[sc.step.output_slots[0]]->as<float>(),
                                            (int)hidden, (int)vocab, scr->cand_val.as<float>(), scr->cand_idx.as<int>(),
                                            scr->cand_cap);
            GemvArgs g;
            g.x = sc.pool[in[0]]->as<float>();
            g.norm_w = sc.pool[in[1]]->as<float>();
            g.eps = eps;
            g.w = sc.pool[in[2]]->ptr();
            g.w_f32 = true;
            g.out = sc.pool[sc.step.output_slots[0]]->as<float>();
            g.K = (int)hidden;
            g.N = (int)vocab;
            g.argmax_val = scr->cand_val.as<float>();
            g.argmax_idx = scr->cand_idx.as<int>();
            g.argmax_cap = scr->cand_cap;
            return gemv_bf16_nk_launch(sc.ctx, g, 1, GEMV_EPI_ARGMAX);
        };
        k.launches.push_back(std::move(h1));
        DeviceLaunch h2;
        h2.name = "finish_step";
        h2.moves_cursor = true;
        h2.bytes_fixed = 64;
        h2.fn = [=](const StepContext &sc) -> int {
            const int ncand = !head_blocks ? std::min(gemv_bf16_nk_grid(sc.ctx, (int)vocab, 4), scr->cand_cap)
                              : head_q6 && head_planes ? q6k_planes_workgroups(sc.ctx, (int)hidden, (int)vocab, scr->cand_cap)
                              : head_k ? gemv_kquant_f32_head_candidates(sc.ctx, head_q6, (int)hidden, (int)vocab, scr->cand_cap)
                              : head_planes ? gemv_planes_workgroups(sc.ctx, head_dt == DType::Q4_0, (int)hidden, (int)vocab)
                                       : gemv_quant_workgroups(sc.ctx, head_dt == DType::Q4_0, (int)hidden, (int)vocab);
            return finish_step_launch(sc.ctx, sc.plan->state(), scr->cand_val.as<float>(),
                                      scr->cand_idx.as<int>(), ncand, sc.plan->out_tokens(),
                                      sc.plan->out_capacity());
        };
        k.launches.push_back(std::move(h2));
        add_step(std::move(k), {ls[L - 1].hidden_out, final_norm, lm_head}, {logits});
    }

    const size_t num_slots = descs.size();
    plan_.reset(new ExecutionPlan(ctx_, std::move(kernels), std::move(steps), num_slots, input_slots,
                                  weight_slots, output_slots, std::move(descs)));
    KvPlanInfo info;
    info.num_layers = L;
    info.num_heads = (int)kvh;
    info.head_dim = (int)hd;
    info.past_kv_input_slots = past_kv;
    info.present_kv_output_slots = present_kv;
    plan_->set_kv_info(info);
    for (int i = 0; i < L; i++) {
        plan_->alias_slot(ls[i].k_out, ls[i].q_out, (size_t)qd * 4);
        plan_->alias_slot(ls[i].v_out, ls[i].q_out, (size_t)(qd + kvd) * 4);
        plan_->alias_slot(ls[i].up_out, ls[i].gate_out, (size_t)inter * 4);
    }
    return HM_OK;
}

// ── running ──────────────────────────────────────────────────────────────────

int HfModel::step_inputs(std::vector<Buffer *> &inputs) {
    inputs = {&ids_view_, &mask_view_, &rope_cos_, &rope_sin_};
    return HM_OK;
}

// The device table of per-layer pointers the whole-step launch reads. It holds the KV cache's
// addresses, so it is rebuilt when the cache has been re-created.
int HfModel::refresh_fused_table() {
    if (!fused_available_ || !plan_ || !plan_->kv_cache()) return HM_OK;
    KvCache *kv = plan_->kv_cache();
    if (fused_table_kv_ == kv->key_ptr(0) && fused_table_max_len_ == kv->max_len()) return HM_OK;
    const int L = cfg_.num_hidden_layers;
    std::vector<FusedLayerPtrs> t((size_t)L);
    for (int l = 0; l < L; l++) {
        const std::string p = "model.layers." + std::to_string(l) + ".";
        FusedLayerPtrs &f = t[l];
        if (fused_wf_ == FUSED_WF_BF16) {
            f.wqkv = packed_[l].qkv.ptr();
            f.wo = packed_[l].o.ptr();
            f.wgu = packed_[l].gate_up.ptr();
            f.wd = packed_[l].down.ptr();
            f.sqkv = f.so = f.sgu = f.sd = nullptr;
        } else if (fused_wf_ == FUSED_WF_K8) {  // byte planes of the four groups, scale records behind them
            const int hidden = cfg_.hidden_size, inter = cfg_.intermediate_size, qd = cfg_.q_dim(), kvd = cfg_.kv_dim();
            auto records = [&](const Buffer &b, int n, int k) {
                return reinterpret_cast<const uint16_t *>(b.as<uint8_t>() + k8_plane_bytes(n, k));
            };
            const LayerPacked &lp = packed_[l];
            f.wqkv = lp.k8[0].ptr();
            f.sqkv = records(lp.k8[0], qd + 2 * kvd, hidden);
            f.wo = lp.k8[1].ptr();
            f.so = records(lp.k8[1], hidden, qd);
            f.wgu = lp.k8[2].ptr();
            f.sgu = records(lp.k8[2], 2 * inter, hidden);
            f.wd = lp.k8[3].ptr();
            f.sd = records(lp.k8[3], hidden, inter);
        } else {  // quant planes of the four runs, scales behind the quants
            const bool q4 = fused_wf_ == FUSED_WF_Q4_0;
            const int hidden = cfg_.hidden_size, inter = cfg_.intermediate_size, qd = cfg_.q_dim(), kvd = cfg_.kv_dim();
            auto scales = [&](const Buffer &b, int n, int k) {
                return reinterpret_cast<const uint16_t *>(b.as<uint8_t>() + quant_planes_scale_offset(q4, n, k));
            };
            const LayerPacked &lp = packed_[l];
            f.wqkv = lp.planes[0].ptr();
            f.sqkv = scales(lp.planes[0], qd + 2 * kvd, hidden);
            f.wo = lp.planes[3].ptr();
            f.so = scales(lp.planes[3], hidden, qd);
            f.wgu = lp.planes[4].ptr();
            f.sgu = scales(lp.planes[4], 2 * inter, hidden);
            f.wd = lp.planes[6].ptr();
            f.sd = scales(lp.planes[6], hidden, inter);
        }
        f.in_ln = weight_f32(p + "input_layernorm.weight");
        f.post_ln = weight_f32(p + "post_attention_layernorm.weight");
        f.q_norm = has_qk_norm_ ? weight_f32(p + "self_attn.q_norm.weight") : nullptr;
        f.k_norm = has_qk_norm_ ? weight_f32(p + "self_attn.k_norm.weight") : nullptr;
        f.qkv_bias = cfg_.attention_bias ? packed_[l].qkv_bias.as<float>() : nullptr;
        f.kcache = kv->key_ptr(l);
        f.vcache = kv->value_ptr(l);
        if (!f.wqkv || !f.wo || !f.wgu || !f.wd || !f.in_ln || !f.post_ln || !f.kcache || !f.vcache)
            return hm_set_error(ctx_, HM_ERR_STATE, "whole-step decode: layer %d has an unset pointer", l);
    }
    int rc = hm_sync(ctx_);  // no launch may still be reading the old table
    if (rc == HM_OK) rc = hm_upload(ctx_, scratch_->fused_layers.ptr(), t.data(), t.size() * sizeof(FusedLayerPtrs));
    if (rc != HM_OK) return rc;
    fused_table_kv_ = kv->key_ptr(0);
    fused_table_max_len_ = kv->max_len();
    return HM_OK;
}

int HfModel::prefill_capture_q8k_inputs(int rows) {
    PrefillScratch &p = pf_;
    int rc = hm_sync(ctx_);
    if (rc != HM_OK) return rc;
    p.capture = Buffer();
    p.capture_rows = 0;
    if (rows <= 0) return HM_OK;
    const TransformerConfig &c = cfg_;
    const size_t per_row = 2 * (size_t)c.hidden_size + (size_t)c.q_dim() + c.intermediate_size;
    const size_t n = (size_t)c.num_hidden_layers * rows * per_row;
    p.capture = Buffer::alloc(ctx_, {(int64_t)n}, DType::F32);
    if (!p.capture) return HM_ERR_OOM;
    HM_HIP(ctx_, hipMemsetAsync(p.capture.ptr(), 0, n * 4, ctx_->stream));
    p.capture_rows = rows;
    p.capture_base = plan_->kv_cache() ? plan_->kv_cache()->current_len() : 0;
    return hm_sync(ctx_);
}

int HfModel::prefill_captured_q8k_inputs(float *h_out, size_t n_floats) {
    PrefillScratch &p = pf_;
    if (!p.capture) return hm_set_error(ctx_, HM_ERR_STATE, "no activation rows were captured");
    if (n_floats * 4 != p.capture.bytes())
        return hm_set_error(ctx_, HM_ERR_INVALID, "captured rows: %zu floats kept, %zu asked for", p.capture.bytes() / 4, n_floats);
    int rc = hm_sync(ctx_);
    if (rc != HM_OK) return rc;
    return hm_download(ctx_, h_out, p.capture.ptr(), n_floats * 4);
}

int HfModel::whole_step_trace(unsigned long long *h_out, int cap, int *n_out) {
    if (!fused_available_) return hm_set_error(ctx_, HM_ERR_STATE, "whole-step decode is not available for this model");
    const int per_wg = cfg_.num_hidden_layers * FUSED_TRACE_PER_LAYER + 2;
    const int all = per_wg * FUSED_TRACE_WGS;
    *n_out = 0;
    int rc = hm_sync(ctx_);
    if (rc != HM_OK) return rc;
    if (!scratch_->fused_trace) {
        scratch_->fused_trace = Buffer::alloc_bytes(ctx_, (size_t)all * 8, {all}, DType::I64);
        if (!scratch_->fused_trace) return HM_ERR_OOM;
        HM_HIP(ctx_, hipMemsetAsync(scratch_->fused_trace.ptr(), 0, (size_t)all * 8, ctx_->stream));
        // a captured step does not know the trace buffer yet
        const bool was = plan_->whole_step();
        if ((rc = plan_->set_whole_step(!was)) != HM_OK || (rc = plan_->set_whole_step(was)) != HM_OK) return rc;
        return hm_sync(ctx_);
    }
    if (cap < per_wg) return hm_set_error(ctx_, HM_ERR_INVALID, "whole_step_trace: room for %d entries, %d needed", cap, per_wg);
    // workgroup 0's row, or every workgroup's rows when there is room for them
    const int n = cap >= all ? all : per_wg;
    rc = hm_download(ctx_, h_out, scratch_->fused_trace.ptr(), (size_t)n * 8);
    if (rc == HM_OK) *n_out = n;
    return rc;
}

// Internal return code of finish_sync: a whole-step launch ran into a wait's bound and the model has been
// switched to one launch per projection; the caller runs its steps again.
constexpr int HM_RETRY_STEPS = -1000;

// Stream sync plus, when steps went through the whole-step launch since the last look, its status words.
int HfModel::finish_sync() {
    int rc = hm_sync(ctx_);
    if (rc != HM_OK || !fused_available_ || !fused_dirty_) return rc;
    fused_dirty_ = false;
    uint32_t h[16] = {0};
    rc = hm_download(ctx_, h, scratch_->fused_ctl.ptr(), sizeof(h));
    return rc == HM_OK ? check_fused_words(h) : rc;
}

// What a host copy of the whole-step control words says: HM_OK, HM_RETRY_STEPS after the recovery from a wait
// that gave up, or the error of a warning, which is reported once.
int HfModel::check_fused_words(const uint32_t *h_ctl) {
    bool gave_up = false;
    const int rc = decode_fused_check_words(ctx_, h_ctl, &gave_up);
    if (rc == HM_OK) return rc;
    if (gave_up) return recover_whole_step();
    (void)hipMemsetAsync(scratch_->fused_ctl.as<uint32_t>() + 3, 0, 4, ctx_->stream);
    (void)hm_sync(ctx_);
    return rc;
}

// After a wait that gave up: keep what the launch reported, clear the exchange area and the control words (the
// launch count with them: tags start over on a zeroed area), and leave the whole-step launch out until the
// caller re-arms it. The grid has drained - every wait is bounded - so nothing is in flight.
int HfModel::recover_whole_step() {
    fused_gave_up_msg_ = ctx_->last_error;
    fused_gave_up_ = true;
    scratch_->inject_spin_limit = 0;
    scratch_->inject_withhold_wg = -1;
    HM_HIP(ctx_, hipMemsetAsync(scratch_->fused_xch.ptr(), 0, scratch_->fused_xch.bytes(), ctx_->stream));
    HM_HIP(ctx_, hipMemsetAsync(scratch_->fused_ctl.ptr(), 0, 64, ctx_->stream));
    int rc = hm_sync(ctx_);
    if (rc == HM_OK) rc = plan_->set_whole_step(false);
    if (rc == HM_OK) rc = plan_->invalidate_graph();
    return rc == HM_OK ? HM_RETRY_STEPS : rc;
}

// Runs `body`; when a whole-step launch inside it gave up a wait, takes the cache back to where the call
// found it and runs the body again, which now takes one launch per projection (rows the failed steps
// appended are written again).
template <class Body>
int HfModel::with_whole_step_retry(Body body) {
    const int len0 = kv_cache_len();
    int rc = body();
    if (rc != HM_RETRY_STEPS) return rc;
    plan_->kv_cache()->reset(len0);
    rc = body();
    return rc == HM_RETRY_STEPS ? hm_set_error(ctx_, HM_ERR_HIP, "whole-step decode gave up twice: %s", fused_gave_up_msg_.c_str()) : rc;
}

int HfModel::set_whole_step(bool on) {
    if (!finalized_) return hm_set_error(ctx_, HM_ERR_STATE, "model not finalized");
    if (on && !fused_available_)
        return hm_set_error(ctx_, HM_ERR_INVALID, "whole-step decode is not available for this model (bf16 weights and a served shape are needed)");
    whole_step_wanted_ = on;
    if (on) fused_gave_up_ = false;  // an explicit request re-arms the launch after a recovered timeout
    return plan_->set_whole_step(on && plan_->kv_cache_len() + 1 <= fused_max_kv_);
}

int HfModel::whole_step_status() {
    if (!fused_available_) return HM_OK;
    if (fused_gave_up_)
        return hm_set_error(ctx_, HM_ERR_HIP, "%s; steps take one launch per projection until reset_kv_cache or set_whole_step(true)",
                            fused_gave_up_msg_.c_str());
    int rc = hm_sync(ctx_);
    if (rc != HM_OK) return rc;
    fused_dirty_ = false;
    bool gave_up = false;
    rc = decode_fused_check(ctx_, scratch_->fused_ctl.as<uint32_t>(), &gave_up);
    if (gave_up && recover_whole_step() == HM_RETRY_STEPS)
        return hm_set_error(ctx_, HM_ERR_HIP, "%s; steps take one launch per projection until reset_kv_cache or set_whole_step(true)",
                            fused_gave_up_msg_.c_str());
    return rc;
}

int HfModel::whole_step_inject_timeout(int workgroup, int spin_limit) {
    if (!fused_available_) return hm_set_error(ctx_, HM_ERR_STATE, "whole-step decode is not available for this model");
    if (workgroup < 0 || spin_limit < 1) return hm_set_error(ctx_, HM_ERR_INVALID, "inject_timeout: workgroup >= 0 and spin_limit >= 1 needed");
    scratch_->inject_spin_limit = spin_limit;
    scratch_->inject_withhold_wg = workgroup;
    return plan_->invalidate_graph();  // a recorded launch carries the old arguments
}

int HfModel::check_ids(const int64_t *ids, int n, std::vector<int32_t> &out) {
    out.resize(n);
    for (int i = 0; i < n; i++) {
        if (ids[i] < 0 || ids[i] >= cfg_.vocab_size)
            return hm_set_error(ctx_, HM_ERR_INVALID, "token id %lld outside the vocabulary (%d)",
                                (long long)ids[i], cfg_.vocab_size);
        out[i] = (int32_t)ids[i];
    }
    return HM_OK;
}

int HfModel::run_kv(const int64_t *h_ids, int n_ids, float *h_logits) {
    if (!finalized_) return hm_set_error(ctx_, HM_ERR_STATE, "model not finalized");
    return with_whole_step_retry([&] { return run_kv_once(h_ids, n_ids, h_logits); });
}

int HfModel::run_kv_once(const int64_t *h_ids, int n_ids, float *h_logits) {
    if (!finalized_) return hm_set_error(ctx_, HM_ERR_STATE, "model not finalized");
    if (n_ids <= 0 || !h_ids) return hm_set_error(ctx_, HM_ERR_INVALID, "run_kv: no input ids");
    if (kv_cache_len() + n_ids > max_seq_len_)
        return hm_set_error(ctx_, HM_ERR_STATE, "KV cache full (%d + %d > %d)", kv_cache_len(), n_ids, max_seq_len_);
    std::vector<int32_t> ids;
    int rc = check_ids(h_ids, n_ids, ids);
    if (rc != HM_OK) return rc;
    if (prefill_min_ > 0 && n_ids >= prefill_min_ && prefill_available()) return prefill(h_ids, n_ids, h_logits);
    if (n_ids > plan_->out_capacity())
        return hm_set_error(ctx_, HM_ERR_INVALID, "run_kv: %d ids exceed the step capacity %d", n_ids, plan_->out_capacity());
    if ((rc = plan_->arm(ids.data(), n_ids)) != HM_OK) return rc;
    std::vector<Buffer *> inputs;
    step_inputs(inputs);
    const size_t logits_slot = plan_->output_slots()[0];
    // The reference's decode loop reads a logits row per token (HfGenerationContext::decode_step,
    // src/hf/model.rs:340-371). The row and the whole-step status words are copied into pinned host memory
    // behind the step, so a token costs one stream synchronisation.
    const size_t row_bytes = (size_t)cfg_.vocab_size * 4;
    if (h_logits && h_stage_bytes_ < row_bytes + 64) {
        if (h_stage_) (void)hipHostFree(h_stage_);
        h_stage_ = nullptr;
        h_stage_bytes_ = 0;
        HM_HIP(ctx_, hipHostMalloc(&h_stage_, row_bytes + 64, hipHostMallocDefault));
        h_stage_bytes_ = row_bytes + 64;
    }
    for (int i = 0; i < n_ids; i++) {
        if ((rc = plan_->run_kv(inputs, weight_bufs_, max_seq_len_)) != HM_OK) return rc;
        if (!h_logits) continue;
        char *stage = static_cast<char *>(h_stage_);
        HM_HIP(ctx_, hipMemcpyAsync(stage, plan_->slot(logits_slot)->ptr(), row_bytes, hipMemcpyDeviceToHost, ctx_->stream));
        const bool look = fused_available_ && fused_dirty_;
        if (look) HM_HIP(ctx_, hipMemcpyAsync(stage + row_bytes, scratch_->fused_ctl.ptr(), 64, hipMemcpyDeviceToHost, ctx_->stream));
        HM_HIP(ctx_, hipStreamSynchronize(ctx_->stream));
        std::memcpy(h_logits + (size_t)i * cfg_.vocab_size, stage, row_bytes);
        if (look) {
            fused_dirty_ = false;
            if ((rc = check_fused_words(reinterpret_cast<const uint32_t *>(stage + row_bytes))) != HM_OK) return rc;
        }
    }
    return finish_sync();
}

// ── prefill pass ─────────────────────────────────────────────────────────────

bool HfModel::prefill_available() const {
    if (!finalized_ || (cfg_.head_dim() != 64 && cfg_.head_dim() != 128)) return false;
    const int hidden = cfg_.hidden_size, qd = cfg_.q_dim(), inter = cfg_.intermediate_size;
    if (weight_dtype_ == DType::BF16) return hidden % 32 == 0 && qd % 32 == 0 && inter % 32 == 0;
    if (!dtype_is_quantized(weight_dtype_)) return false;
    // Block formats: K tiles of 64; the matrices that share an activation (q|k|v, gate|up) must agree
    // on what they multiply with, f32 rows (Q8_0, Q4_0) or Q8_K rows (the K-quants).
    if (hidden % 64 != 0 || qd % 64 != 0 || inter % 64 != 0) return false;
    auto kq = [&](int l, int j) { const DType t = proj_dtype(l, j); return t == DType::Q4_K || t == DType::Q6_K; };
    for (int l = 0; l < cfg_.num_hidden_layers; l++) {
        if (kq(l, 0) != kq(l, 1) || kq(l, 0) != kq(l, 2) || kq(l, 4) != kq(l, 5)) return false;
        if (((kq(l, 0) || kq(l, 4)) && hidden % 256 != 0) || (kq(l, 3) && qd % 256 != 0) || (kq(l, 6) && inter % 256 != 0))
            return false;
    }
    return true;
}

void HfModel::set_prefill_weight_cache(size_t bytes) {
    prefill_weight_cache_bytes_ = bytes;
    if (ctx_) hm_sync(ctx_);
    pf_.wcache.clear();
}

const float *HfModel::weight_f32(const std::string &name) const {
    auto it = slot_by_name_.find(name);
    return it == slot_by_name_.end() ? nullptr : weight_bufs_[it->second].as<float>();
}

int HfModel::prefill(const int64_t *h_ids, int n_ids, float *h_logits) {
    if (!finalized_) return hm_set_error(ctx_, HM_ERR_STATE, "model not finalized");
    if (!prefill_available())
        return hm_set_error(ctx_, HM_ERR_INVALID, "prefill: needs head_dim 64 or 128 and widths that are multiples of 32 (bf16) or 64 (block formats, whose q|k|v and gate|up must each be of one kind)");
    if (n_ids <= 0 || !h_ids) return hm_set_error(ctx_, HM_ERR_INVALID, "prefill: no input ids");
    if (kv_cache_len() + n_ids > max_seq_len_)
        return hm_set_error(ctx_, HM_ERR_STATE, "KV cache full (%d + %d > %d)", kv_cache_len(), n_ids, max_seq_len_);
    std::vector<int32_t> ids;
    int rc = check_ids(h_ids, n_ids, ids);
    if (rc != HM_OK) return rc;
    constexpr int CHUNK = 512;
    for (int at = 0; at < n_ids; at += CHUNK) {
        const int n = std::min(CHUNK, n_ids - at);
        rc = prefill_chunk(ids.data() + at, n, h_logits ? h_logits + (size_t)at * cfg_.vocab_size : nullptr);
        if (rc != HM_OK) return rc;
    }
    return hm_sync(ctx_);
}

int HfModel::prefill_chunk(const int32_t *h_ids, int n, float *h_logits) {
    const TransformerConfig &c = cfg_;
    const int hidden = c.hidden_size, inter = c.intermediate_size, vocab = c.vocab_size;
    const int H = c.num_attention_heads, kvh = c.kv_heads(), hd = c.head_dim();
    const int qd = c.q_dim(), kvd = c.kv_dim(), nqkv = qd + 2 * kvd;
    const float eps = (float)c.rms_norm_eps;
    PrefillScratch &p = pf_;
    const bool quant = dtype_is_quantized(weight_dtype_);
    if (p.rows < n) {
        const int rows = std::max(n, 128);
        const int64_t widest = std::max<int64_t>(std::max(hidden, qd), inter);
        hm_sync(ctx_);
        {
            PrefillScratch grown;  // a capture that a test switched on outlives the regrowth
            grown.capture = std::move(p.capture);
            grown.capture_rows = p.capture_rows;
            grown.capture_base = p.capture_base;
            grown.icache = std::move(p.icache);  // weights, not rows: they do not depend on the chunk size
            grown.icache_off = p.icache_off;
            grown.scache = std::move(p.scache);
            grown.scache_off = p.scache_off;
            p = std::move(grown);
        }
        p.ids = Buffer::alloc(ctx_, {rows}, DType::F32);  // int32 ids
        p.h = Buffer::alloc(ctx_, {rows, hidden}, DType::F32);
        p.resid = Buffer::alloc(ctx_, {rows, hidden}, DType::F32);
        p.split = Buffer::alloc(ctx_, {rows, 3 * widest}, DType::BF16);
        p.qkv = Buffer::alloc(ctx_, {PrefillScratch::MAX_PARTS, rows, nqkv}, DType::F32);
        p.proj_out = Buffer::alloc(ctx_, {PrefillScratch::MAX_PARTS, rows, hidden}, DType::F32);
        p.gate_up = Buffer::alloc(ctx_, {PrefillScratch::MAX_PARTS, rows, 2 * (int64_t)inter}, DType::F32);
        if (!p.ids || !p.h || !p.resid || !p.split || !p.qkv || !p.proj_out || !p.gate_up) return HM_ERR_OOM;
        if (quant && widest % 256 == 0) {  // Q8_K rows for K-quant groups (a float holds four of the int8 values)
            p.q8 = Buffer::alloc(ctx_, {rows, widest / 4}, DType::F32);
            p.q8s = Buffer::alloc(ctx_, {rows, widest / 256}, DType::F32);
            if (!p.q8 || !p.q8s) return HM_ERR_OOM;
        }
        if (quant) {  // the largest group of matrices of a layer as three bf16 pieces per weight
            const int64_t most = std::max(std::max((int64_t)nqkv * hidden, (int64_t)hidden * qd), 2 * (int64_t)inter * hidden);
            p.wsplit = Buffer::alloc(ctx_, {3 * most}, DType::BF16);
            if (!p.wsplit) return HM_ERR_OOM;
        }
        p.rows = rows;
    }
    if (h_logits && !p.logits) {
        p.logits = Buffer::alloc(ctx_, {p.rows, vocab}, DType::F32);
        if (!p.logits) return HM_ERR_OOM;
    }
    KvCache *kv = plan_->kv_cache();
    const int past = kv->current_len();
    int rc = hm_upload(ctx_, p.ids.ptr(), h_ids, (size_t)n * 4);
    if (rc != HM_OK) return rc;
    float *h = p.h.as<float>(), *resid = p.resid.as<float>(), *qkv = p.qkv.as<float>();
    float *proj_out = p.proj_out.as<float>(), *gate_up = p.gate_up.as<float>();
    uint16_t *split = p.split.as<uint16_t>();
    const int np = quant ? 3 : prefill_pieces_;
    const int MP = PrefillScratch::MAX_PARTS;
    int parts = 1;  // K slices of the latest projection
    uint16_t *wsplit = quant ? p.wsplit.as<uint16_t>() : nullptr;
    static const char *const proj_name[7] = {"self_attn.q_proj.weight", "self_attn.k_proj.weight", "self_attn.v_proj.weight",
                                             "self_attn.o_proj.weight", "mlp.gate_proj.weight", "mlp.up_proj.weight",
                                             "mlp.down_proj.weight"};
    const int proj_n[7] = {qd, kvd, kvd, hidden, inter, inter, hidden};
    // K-quant matrices multiply with Q8_K rows (reference emit_quant.rs:422-466), everything else with the f32 rows
    auto q8k = [&](int l, int which) {
        const DType t = proj_dtype(l, which);
        return quant && (t == DType::Q4_K || t == DType::Q6_K);
    };
    // out[n][N] (N = the members' rows together) = split x W^T for the projections first .. first + count - 1
    // of layer l, which share the activation in `split`. bf16: the packed stream matrix. Block formats
    // (reference emit_quant_matmul_kernel, src/hf/emitter_quant.rs:675-702): the members are
    // dequantised into wsplit one under the other, or row-interleaved for gate|up, which is the order
    // the packed bf16 matrices have.
    // Resident pieces: when six bytes per projection weight fit the budget (and leave an eighth of the
    // device free), each group's matrix is dequantised on first use and kept.
    if (quant && p.wcache.empty() && prefill_weight_cache_bytes_ > 0) {
        const size_t per_layer = ((size_t)nqkv * hidden + (size_t)hidden * qd + 3 * (size_t)inter * hidden) * 6;
        size_t free_b = 0, total_b = 0;
        if (hipMemGetInfo(&free_b, &total_b) != hipSuccess) free_b = total_b = 0;
        const size_t need = per_layer * c.num_hidden_layers;
        if (need <= prefill_weight_cache_bytes_ && need + total_b / 8 <= free_b) p.wcache.resize((size_t)c.num_hidden_layers * 4);
    }
    // K-quant groups multiply on the integer matrix cores (gemm_kquant_i8.h) when their digit planes
    // (3 bytes a weight) fit the same budget: packed on first use, resident afterwards.
    if (quant && p.icache.empty() && !p.icache_off && p.q8 && prefill_weight_cache_bytes_ > 0) {
        size_t need = 0;
        const int gK[4] = {hidden, qd, hidden, inter}, gN[4] = {nqkv, hidden, 2 * inter, hidden}, gfirst[4] = {0, 3, 4, 6};
        for (int l = 0; l < c.num_hidden_layers; l++)
            for (int gq = 0; gq < 4; gq++)
                if (q8k(l, gfirst[gq]) && gK[gq] % 256 == 0 && gK[gq] / 256 <= 16 * MP)
                    need += kq_i8_plane_bytes(gN[gq], gK[gq]) + kq_i8_scale_bytes(gN[gq], gK[gq]) + 256;
        size_t free_b = 0, total_b = 0;
        if (hipMemGetInfo(&free_b, &total_b) != hipSuccess) free_b = total_b = 0;
        if (need > 0 && need <= prefill_weight_cache_bytes_ && need + total_b / 8 <= free_b)
            p.icache.resize((size_t)c.num_hidden_layers * 4);
        else
            p.icache_off = true;
    }
    // the planes of group g (0 q|k|v, 1 o, 2 gate|up, 3 down) of layer l, packed now if this is their first use;
    // nullptr: the group goes through the bf16 pieces
    auto i8_planes = [&](int l, int g, int first, int count, int K) -> const Buffer * {
        if (p.icache.empty() || !q8k(l, first) || K % 256 != 0 || K / 256 > 16 * MP) return nullptr;
        Buffer &slot = p.icache[(size_t)l * 4 + g];
        if (slot) return &slot;
        int N = 0;
        for (int j = first; j < first + count; j++) N += proj_n[j];
        const size_t pb = (kq_i8_plane_bytes(N, K) + 255) / 256 * 256, sb = kq_i8_scale_bytes(N, K);
        slot = Buffer::alloc(ctx_, {(int64_t)((pb + sb + 3) / 4)}, DType::F32);
        if (!slot) {
            (void)hipGetLastError();
            return nullptr;
        }
        const bool interleave = first == 4 && count == 2;
        int8_t *planes = slot.as<int8_t>();
        float *scales = reinterpret_cast<float *>(slot.as<char>() + pb);
        int row = 0;
        for (int j = first; j < first + count; j++) {
            auto it = slot_by_name_.find("model.layers." + std::to_string(l) + "." + proj_name[j]);
            int rc2 = it == slot_by_name_.end() ? HM_ERR_STATE : HM_OK;
            if (rc2 == HM_OK)
                rc2 = kq_i8_pack(ctx_, (int)proj_dtype(l, j), weight_bufs_[it->second].as<uint8_t>(), proj_n[j], K,
                                 interleave ? planes : planes + (size_t)row * K,
                                 interleave ? scales : scales + (size_t)row * (K / 256) * 2, N, interleave ? 2 : 1,
                                 interleave ? j - first : 0);
            if (rc2 != HM_OK) {
                slot = Buffer();
                return nullptr;
            }
            row += proj_n[j];
        }
        return &slot;
    };
    // Q8_0 / Q4_0 groups multiply their integers (bf16, exact) and apply the block scales in the GEMM
    // (2 bytes a weight + the scales), under the same budget; otherwise the dequantised weights as bf16 pieces.
    auto plain_block = [&](int l, int which) {
        const DType t = proj_dtype(l, which);
        return quant && (t == DType::Q8_0 || t == DType::Q4_0);
    };
    if (quant && p.scache.empty() && !p.scache_off && prefill_weight_cache_bytes_ > 0) {
        size_t need = 0;
        const int gK[4] = {hidden, qd, hidden, inter}, gN[4] = {nqkv, hidden, 2 * inter, hidden}, gfirst[4] = {0, 3, 4, 6};
        for (int l = 0; l < c.num_hidden_layers; l++)
            for (int gq = 0; gq < 4; gq++)
                if (plain_block(l, gfirst[gq]))
                    need += (size_t)gN[gq] * gK[gq] * 2 + (size_t)(gK[gq] / 32) * (gN[gq] + 127) * 4 + 512;
        size_t free_b = 0, total_b = 0;
        if (hipMemGetInfo(&free_b, &total_b) != hipSuccess) free_b = total_b = 0;
        if (need > 0 && need <= prefill_weight_cache_bytes_ && need + total_b / 8 <= free_b)
            p.scache.resize((size_t)c.num_hidden_layers * 4);
        else
            p.scache_off = true;
    }
    auto scaled_ints = [&](int l, int g, int first, int count, int K, int *npad_out) -> const Buffer * {
        if (p.scache.empty()) return nullptr;
        for (int j = first; j < first + count; j++)
            if (!plain_block(l, j)) return nullptr;
        int N = 0;
        for (int j = first; j < first + count; j++) N += proj_n[j];
        const int npad = (N + 127) / 128 * 128;
        *npad_out = npad;
        Buffer &slot = p.scache[(size_t)l * 4 + g];
        if (slot) return &slot;
        const size_t ib = ((size_t)N * K * 2 + 255) / 256 * 256, sb = (size_t)(K / 32) * npad * 4;
        slot = Buffer::alloc(ctx_, {(int64_t)((ib + sb + 3) / 4)}, DType::F32);
        if (!slot) {
            (void)hipGetLastError();
            return nullptr;
        }
        const bool interleave = first == 4 && count == 2;
        uint16_t *ints = slot.as<uint16_t>();
        float *scales = reinterpret_cast<float *>(slot.as<char>() + ib);
        int row = 0;
        for (int j = first; j < first + count; j++) {
            auto it = slot_by_name_.find("model.layers." + std::to_string(l) + "." + proj_name[j]);
            int rc2 = it == slot_by_name_.end() ? HM_ERR_STATE : HM_OK;
            if (rc2 == HM_OK)
                rc2 = quant_ints_launch(ctx_, (int)proj_dtype(l, j), weight_bufs_[it->second].as<uint8_t>(), proj_n[j], K,
                                        interleave ? ints : ints + (size_t)row * K, interleave ? scales : scales + row, npad,
                                        interleave ? 2 : 1, interleave ? j - first : 0);
            if (rc2 != HM_OK) {
                slot = Buffer();
                return nullptr;
            }
            row += proj_n[j];
        }
        return &slot;
    };
    const Buffer *i8 = nullptr;  // the planes of the group about to be multiplied, if it takes that path
    int8_t *q8 = p.q8 ? p.q8.as<int8_t>() : nullptr;
    float *q8s = p.q8s ? p.q8s.as<float>() : nullptr;
    auto project = [&](int l, int first, int count, const Buffer &packed, int K, float *out) -> int {
        int N = 0;
        for (int j = first; j < first + count; j++) N += proj_n[j];
        if (!quant) return gemm_split_nk(ctx_, split, np, packed.as<uint16_t>(), out, n, K, N, MP, &parts);
        if (i8) {
            const size_t pb = (kq_i8_plane_bytes(N, K) + 255) / 256 * 256;
            return gemm_q8k_kquant_nk(ctx_, q8, q8s, i8->as<int8_t>(), reinterpret_cast<const float *>(i8->as<char>() + pb), out, n,
                                      K, N, MP, &parts);
        }
        {
            int npad = 0;
            const int g = first == 0 ? 0 : first == 3 ? 1 : first == 4 ? 2 : 3;
            if (const Buffer *sc = scaled_ints(l, g, first, count, K, &npad)) {
                const size_t ib = ((size_t)N * K * 2 + 255) / 256 * 256;
                return gemm_pieces_scaled_nk(ctx_, split, sc->as<uint16_t>(), reinterpret_cast<const float *>(sc->as<char>() + ib),
                                             npad, out, n, K, N, MP, &parts);
            }
        }
        const bool interleave = first == 4 && count == 2;
        uint16_t *wsplit = p.wsplit.as<uint16_t>();
        if (!p.wcache.empty()) {
            Buffer &slot = p.wcache[(size_t)l * 4 + (first == 0 ? 0 : first == 3 ? 1 : first == 4 ? 2 : 3)];
            if (slot) return gemm_split_split_nk(ctx_, split, slot.as<uint16_t>(), out, n, K, N, MP, &parts);
            slot = Buffer::alloc(ctx_, {(int64_t)N, 3 * (int64_t)K}, DType::BF16);
            if (slot)
                wsplit = slot.as<uint16_t>();
            else
                (void)hipGetLastError();  // out of memory: this group keeps using the scratch matrix
        }
        int row = 0;
        for (int j = first; j < first + count; j++) {
            auto it = slot_by_name_.find("model.layers." + std::to_string(l) + "." + proj_name[j]);
            if (it == slot_by_name_.end()) return hm_set_error(ctx_, HM_ERR_STATE, "prefill: weight %s missing", proj_name[j]);
            const int rc = dequant_split_launch(ctx_, (int)proj_dtype(l, j), weight_bufs_[it->second].as<uint8_t>(), proj_n[j], K,
                                                interleave ? wsplit : wsplit + (size_t)row * 3 * K, interleave ? 2 : 1,
                                                interleave ? j - first : 0);
            if (rc != HM_OK) return rc;
            row += proj_n[j];
        }
        return gemm_split_split_nk(ctx_, split, wsplit, out, n, K, N, MP, &parts);
    };
    rc = embed_launch(ctx_, nullptr, p.ids.as<int32_t>(), weight_f32("model.embed_tokens.weight"), h, n, vocab, hidden);
    if (rc != HM_OK) return rc;
    // where (layer, group)'s rows of this chunk go in the capture buffer, or nullptr
    auto capture_at = [&](int l, int group) -> float * {
        if (!p.capture) return nullptr;
        const int r0 = past - p.capture_base;
        if (r0 < 0 || r0 + n > p.capture_rows) return nullptr;
        const size_t R = (size_t)p.capture_rows;
        const size_t goff[4] = {0, R * hidden, R * (hidden + qd), R * (2 * (size_t)hidden + qd)};
        const size_t gdim[4] = {(size_t)hidden, (size_t)qd, (size_t)hidden, (size_t)inter};
        return p.capture.as<float>() + (size_t)l * R * (2 * (size_t)hidden + qd + inter) + goff[group] + (size_t)r0 * gdim[group];
    };
    // The hidden state entering a layer is x [+ res]: the embedding for the first layer, afterwards the
    // post-attention residual plus the K slices of the previous down projection, which the next
    // RMSNorm kernel adds on its way (the reference's ResAdd, src/hf/emitter.rs:804).
    const float *x = h, *res = nullptr;
    int res_parts = 1;
    for (int l = 0; l < c.num_hidden_layers; l++) {
        const std::string pre = "model.layers." + std::to_string(l) + ".";
        const LayerPacked &lp = packed_[l];
        // QKV kernel (reference src/hf/emitter.rs:549-673)
        i8 = i8_planes(l, 0, 0, 3, hidden);
        rc = rmsnorm_split_launch(ctx_, x, res, res_parts, weight_f32(pre + "input_layernorm.weight"), split, np,
                                  res ? h : nullptr, n, hidden, eps, q8k(l, 0), q8k(l, 0) ? capture_at(l, 0) : nullptr,
                                  i8 ? q8 : nullptr, i8 ? q8s : nullptr);
        if (rc == HM_OK) rc = project(l, 0, 3, lp.qkv, hidden, qkv);
        if (rc != HM_OK) return rc;
        QkvPostArgs qa;
        qa.qkv = qkv;
        qa.parts = parts;
        qa.part_stride = (size_t)n * nqkv;
        qa.bias = lp.qkv_bias ? lp.qkv_bias.as<float>() : nullptr;
        if (has_qk_norm_) {
            qa.qw = weight_f32(pre + "self_attn.q_norm.weight");
            qa.kw = weight_f32(pre + "self_attn.k_norm.weight");
        }
        qa.cos_tab = rope_cos_.as<float>();
        qa.sin_tab = rope_sin_.as<float>();
        qa.kcache = kv->key_ptr(l);
        qa.vcache = kv->value_ptr(l);
        qa.S = n;
        qa.H = H;
        qa.kvh = kvh;
        qa.hd = hd;
        qa.max_len = kv->max_len();
        qa.past = past;
        qa.eps = eps;
        if ((rc = qkv_post_launch(ctx_, qa)) != HM_OK) return rc;
        // attention kernel (reference src/hf/emitter.rs:683-758): causal attention, then the O projection
        PrefillAttnArgs aa;
        aa.q = qkv;
        aa.ldq = nqkv;
        aa.kcache = kv->key_ptr(l);
        aa.vcache = kv->value_ptr(l);
        // a K-quant O projection wants whole rows for its Q8_K blocks: the heads' outputs go out as f32
        // (into the idle gate|up scratch) and are split afterwards
        const bool o_q8k = q8k(l, 3);
        if (o_q8k)
            aa.out_f32 = gate_up;
        else
            aa.out_split = split;
        aa.S = n;
        aa.H = H;
        aa.kvh = kvh;
        aa.hd = hd;
        aa.max_len = kv->max_len();
        aa.past = past;
        aa.scale = (float)(1.0 / std::sqrt((double)hd));
        aa.pieces = np;
        if ((rc = prefill_attn_launch(ctx_, aa)) != HM_OK) return rc;
        i8 = i8_planes(l, 1, 3, 1, qd);
        if (o_q8k && i8 && (rc = quantize_q8k_rows_launch(ctx_, gate_up, q8, q8s, (size_t)n, qd)) != HM_OK) return rc;
        if (o_q8k && !i8 && (rc = split_rows_launch(ctx_, gate_up, split, np, (size_t)n, qd, true)) != HM_OK) return rc;
        if (o_q8k && capture_at(l, 1))
            HM_HIP(ctx_, hipMemcpyAsync(capture_at(l, 1), gate_up, (size_t)n * qd * 4, hipMemcpyDeviceToDevice, ctx_->stream));
        if ((rc = project(l, 3, 1, lp.o, qd, proj_out)) != HM_OK) return rc;
        // MLP kernel (reference src/hf/emitter.rs:767-822); h holds the layer's input by now
        i8 = i8_planes(l, 2, 4, 2, hidden);
        rc = rmsnorm_split_launch(ctx_, h, proj_out, parts, weight_f32(pre + "post_attention_layernorm.weight"), split, np,
                                  resid, n, hidden, eps, q8k(l, 4), q8k(l, 4) ? capture_at(l, 2) : nullptr,
                                  i8 ? q8 : nullptr, i8 ? q8s : nullptr);
        if (rc == HM_OK) rc = project(l, 4, 2, lp.gate_up, hidden, gate_up);
        i8 = i8_planes(l, 3, 6, 1, inter);
        if (rc == HM_OK) rc = silu_mul_split_launch(ctx_, gate_up, parts, split, np, n, inter, q8k(l, 6), q8k(l, 6) ? capture_at(l, 3) : nullptr,
                                                    i8 ? q8 : nullptr, i8 ? q8s : nullptr);
        if (rc == HM_OK) rc = project(l, 6, 1, lp.down, inter, proj_out);
        i8 = nullptr;
        if (rc != HM_OK) return rc;
        x = resid;
        res = proj_out;
        res_parts = parts;
    }
    if (h_logits) {  // LM head (reference src/hf/emitter.rs:828-862) for every row
        rc = rmsnorm_split_launch(ctx_, x, res, res_parts, weight_f32("model.norm.weight"), split, np, nullptr, n, hidden, eps);
        if (rc == HM_OK && !quant)
            rc = gemm_split_nk(ctx_, split, np, lm_head_packed_.as<uint16_t>(), p.logits.as<float>(), n, hidden, vocab);
        if (rc == HM_OK && quant) {
            // the quantised plan's LM head is f32 [vocab][hidden] (reference src/hf/emitter_quant.rs:1390-1437):
            // slabs of its rows become bf16 pieces in wsplit, as many as fit
            const int slab = (int)std::min<int64_t>(vocab, (int64_t)(p.wsplit.bytes() / 2) / (3 * (int64_t)hidden) / 128 * 128);
            if (slab <= 0) return hm_set_error(ctx_, HM_ERR_STATE, "prefill: weight scratch too small for the LM head");
            const size_t head_rowbytes = lm_head_blocks_ ? lm_head_blocks_.bytes() / (size_t)vocab : 0;
            for (int v0 = 0; v0 < vocab && rc == HM_OK; v0 += slab) {
                const int rows = std::min(slab, vocab - v0);
                if (lm_head_blocks_)  // rows of the output matrix dequantised from its blocks (bit-exact) into the pieces
                    rc = dequant_split_launch(ctx_, (int)lm_head_blocks_dtype_, lm_head_blocks_.as<uint8_t>() + (size_t)v0 * head_rowbytes,
                                              rows, (int)hidden, wsplit, 1, 0);
                else
                    rc = split_rows_launch(ctx_, lm_head_packed_.as<float>() + (size_t)v0 * hidden, wsplit, 3, (size_t)rows, hidden);
                if (rc == HM_OK)
                    rc = gemm_split_split_nk(ctx_, split, wsplit, p.logits.as<float>() + v0, n, hidden, rows, 1, nullptr, vocab);
            }
        }
        if (rc == HM_OK) rc = hm_download(ctx_, h_logits, p.logits.ptr(), (size_t)n * vocab * 4);
        if (rc != HM_OK) return rc;
    }
    // one advance after all layers appended (reference src/runtime.rs:1875-1880)
    kv->advance_by(n);
    return HM_OK;
}

int HfModel::init_kv_cache(const float *const *h_kv, int seq_len) {
    if (!finalized_) return hm_set_error(ctx_, HM_ERR_STATE, "model not finalized");
    return plan_->init_kv_cache(h_kv, seq_len, max_seq_len_);
}

int HfModel::reset_kv_cache() {
    if (!finalized_) return hm_set_error(ctx_, HM_ERR_STATE, "model not finalized");
    plan_->reset_kv_cache();
    fused_gave_up_ = false;  // a new conversation re-arms the whole-step launch after a recovered timeout
    return HM_OK;
}

int HfModel::kv_cache_len() const { return plan_ ? plan_->kv_cache_len() : 0; }

int HfModel::generate_greedy(const int64_t *h_prompt, int n_prompt, int n_new, int32_t *h_tokens) {
    if (!finalized_) return hm_set_error(ctx_, HM_ERR_STATE, "model not finalized");
    return with_whole_step_retry([&] { return generate_greedy_once(h_prompt, n_prompt, n_new, h_tokens); });
}

int HfModel::generate_greedy_once(const int64_t *h_prompt, int n_prompt, int n_new, int32_t *h_tokens) {
    if (!finalized_) return hm_set_error(ctx_, HM_ERR_STATE, "model not finalized");
    if (n_prompt <= 0 || n_new <= 0 || !h_prompt || !h_tokens)
        return hm_set_error(ctx_, HM_ERR_INVALID, "generate_greedy: bad arguments");
    int steps = n_prompt + n_new - 1;
    if (kv_cache_len() + steps > max_seq_len_)  // the reference's loop stops at max_seq_len
                                                // (src/generate.rs:188-194); here it is an error
        return hm_set_error(ctx_, HM_ERR_STATE, "KV cache full (%d + %d > %d)", kv_cache_len(), steps, max_seq_len_);
    if (prefill_min_ > 0 && n_prompt - 1 >= prefill_min_ && prefill_available()) {
        // reference HfGenerationContext::prefill (src/hf/model.rs:321-336): the prompt in one pass; its
        // last token goes through the decode step, whose pick is generated token 0
        int rc = prefill(h_prompt, n_prompt - 1, nullptr);
        if (rc != HM_OK) return rc;
        h_prompt += n_prompt - 1;
        n_prompt = 1;
        steps = n_new;
    }
    if (steps > plan_->out_capacity())
        return hm_set_error(ctx_, HM_ERR_INVALID, "generate_greedy: %d steps exceed capacity %d", steps, plan_->out_capacity());
    std::vector<int32_t> ids;
    int rc = check_ids(h_prompt, n_prompt, ids);
    if (rc != HM_OK) return rc;
    if ((rc = plan_->arm(ids.data(), n_prompt)) != HM_OK) return rc;
    std::vector<Buffer *> inputs;
    step_inputs(inputs);
    for (int i = 0; i < steps; i++)
        if ((rc = plan_->run_kv(inputs, weight_bufs_, max_seq_len_)) != HM_OK) return rc;
    // the pick after prompt token n_prompt-1 is generated token 0
    rc = hm_download(ctx_, h_tokens, plan_->out_tokens() + (n_prompt - 1), (size_t)n_new * 4);
    return rc == HM_OK ? finish_sync() : rc;
}

// sampling.hip
int sample_check_config(hm_ctx *ctx, const hm_sampling_config *cfg, bool device);
int sample_token_launch(hm_ctx *ctx, const float *d_logits, float *d_work, const int *d_counts, int vocab,
                        const hm_sampling_config &cfg, float draw, int32_t *d_out, int *d_counts_update, int32_t *d_list,
                        int list_pos);
int sample_step_launch(hm_ctx *ctx, const float *d_logits, float *d_work, int *d_counts, int vocab,
                       const hm_sampling_config &cfg, DecodeState *d_cursor, const float *d_draws, int32_t *d_list,
                       int eos, int *d_stop, int32_t *d_out);
int zero_ints_launch(hm_ctx *ctx, int *d, size_t n);

int HfModel::generate(const int64_t *h_prompt, int n_prompt, int max_new, const hm_sampling_config &cfg, uint64_t seed,
                      int eos_token, int32_t *h_tokens, int *n_out) {
    if (!finalized_) return hm_set_error(ctx_, HM_ERR_STATE, "model not finalized");
    return with_whole_step_retry([&] { return generate_once(h_prompt, n_prompt, max_new, cfg, seed, eos_token, h_tokens, n_out); });
}

int HfModel::generate_once(const int64_t *h_prompt, int n_prompt, int max_new, const hm_sampling_config &cfg, uint64_t seed,
                           int eos_token, int32_t *h_tokens, int *n_out) {
    if (!finalized_) return hm_set_error(ctx_, HM_ERR_STATE, "model not finalized");
    if (n_prompt <= 0 || max_new <= 0 || !h_prompt || !h_tokens || !n_out)
        return hm_set_error(ctx_, HM_ERR_INVALID, "generate: bad arguments");
    *n_out = 0;
    const bool greedy = cfg.temperature <= 0.0f;
    const bool on_device = greedy || (cfg.top_k >= 1 && cfg.top_k <= 1024);
    int rc = sample_check_config(ctx_, &cfg, on_device);
    if (rc != HM_OK) return rc;
    if (kv_cache_len() + n_prompt > max_seq_len_)
        return hm_set_error(ctx_, HM_ERR_STATE, "KV cache full (%d + %d > %d)", kv_cache_len(), n_prompt, max_seq_len_);
    std::vector<int32_t> ids;
    if ((rc = check_ids(h_prompt, n_prompt, ids)) != HM_OK) return rc;
    const int vocab = cfg_.vocab_size;
    SamplerScratch &s = sampler_;
    if (!s.work) {
        s.work = Buffer::alloc(ctx_, {vocab}, DType::F32);
        s.counts = Buffer::alloc(ctx_, {vocab}, DType::F32);  // int32 counts
        s.token = Buffer::alloc(ctx_, {64}, DType::F32);
        if (!s.work || !s.counts || !s.token) return HM_ERR_OOM;
    }
    if (s.list_cap < max_new) {
        s.list = Buffer::alloc(ctx_, {max_new}, DType::F32);  // int32 token list
        if (!s.list) return HM_ERR_OOM;
        s.list_cap = max_new;
    }
    const bool penalties = cfg.repetition_penalty != 1.0f || cfg.frequency_penalty != 0.0f || cfg.presence_penalty != 0.0f;
    if ((rc = zero_ints_launch(ctx_, s.counts.as<int>(), (size_t)vocab)) != HM_OK) return rc;
    // prompt: everything but its last token only has to reach the cache
    // (reference HfGenerationContext::prefill, src/hf/model.rs:321-336)
    if (n_prompt > 1) {
        if ((rc = run_kv_once(h_prompt, n_prompt - 1, nullptr)) != HM_OK) return rc;
    }
    uint64_t rng = hm_rng_seed(seed);
    std::vector<Buffer *> inputs;
    step_inputs(inputs);
    const size_t logits_slot = plan_->output_slots()[0];
    std::vector<float> host_logits;
    std::vector<uint32_t> generated;
    int32_t current = ids[n_prompt - 1];
    if (on_device) {
        // Device-resident loop: steps are enqueued in chunks with nothing read back in between. The step's
        // own pick (greedy, no penalties) or the sampler launched behind it (its draw taken from a list made
        // up front, its pick written over the cursor's next input) feeds the next step on the GPU; the host
        // reads a chunk's tokens once, and on an end-of-sequence token takes the cache back to the row of the
        // step that produced it (the reference stops there: src/generate.rs:231-246).
        const bool own_pick = greedy && !penalties;
        if (!greedy) {
            std::vector<float> draws((size_t)max_new);
            for (auto &d : draws) d = hm_rng_next_f32(&rng);
            if (s.draws_cap < max_new) {
                s.draws = Buffer::alloc(ctx_, {max_new}, DType::F32);
                if (!s.draws) return HM_ERR_OOM;
                s.draws_cap = max_new;
            }
            if ((rc = hm_upload(ctx_, s.draws.ptr(), draws.data(), draws.size() * 4)) != HM_OK) return rc;
        }
        const int chunk_cap = std::min(plan_->out_capacity(), 16);
        std::vector<int32_t> got((size_t)chunk_cap);
        int done = 0;
        while (done < max_new) {
            const int len0 = kv_cache_len();
            const int n = std::min({chunk_cap, max_new - done, max_seq_len_ - len0});
            if (n <= 0) break;  // context limit (src/generate.rs:188-194)
            if ((rc = plan_->arm(&current, 1)) != HM_OK) return rc;
            int32_t *d_stop = s.token.as<int32_t>() + 1;
            const int32_t minus_one = -1;
            if (!own_pick && (rc = hm_upload(ctx_, d_stop, &minus_one, 4)) != HM_OK) return rc;
            for (int i = 0; i < n; i++) {
                if ((rc = plan_->run_kv(inputs, weight_bufs_, max_seq_len_)) != HM_OK) return rc;
                if (own_pick) continue;
                rc = sample_step_launch(ctx_, plan_->slot(logits_slot)->as<float>(), s.work.as<float>(),
                                        penalties ? s.counts.as<int>() : nullptr, vocab, cfg, plan_->state(),
                                        greedy ? nullptr : s.draws.as<float>() + done, s.list.as<int32_t>() + done, eos_token,
                                        d_stop, s.token.as<int32_t>());
                if (rc != HM_OK) return rc;
            }
            rc = hm_download(ctx_, got.data(), own_pick ? plan_->out_tokens() : s.list.as<int32_t>() + done, (size_t)n * 4);
            if (rc != HM_OK) return rc;
            int taken = n;
            for (int i = 0; i < n; i++)
                if (got[i] == eos_token) {
                    taken = i;
                    break;
                }
            for (int i = 0; i < taken; i++) h_tokens[(*n_out)++] = got[i];
            if (taken < n) {
                plan_->kv_cache()->reset(len0 + taken + 1);  // rows of the steps behind the stop are dropped
                break;
            }
            current = got[n - 1];
            done += n;
        }
        return finish_sync();
    }
    for (int step = 0; step < max_new; step++) {
        if (kv_cache_len() >= max_seq_len_) break;  // context limit (src/generate.rs:188-194)
        if ((rc = plan_->arm(&current, 1)) != HM_OK) return rc;
        if ((rc = plan_->run_kv(inputs, weight_bufs_, max_seq_len_)) != HM_OK) return rc;
        const float *d_logits = plan_->slot(logits_slot)->as<float>();
        int32_t tok = 0;
        host_logits.resize(vocab);
        rc = hm_download(ctx_, host_logits.data(), d_logits, (size_t)vocab * 4);
        if (rc == HM_OK)
            rc = hm_sample_token_host(host_logits.data(), vocab, &cfg, generated.data(), (int)generated.size(), &rng, &tok);
        if (rc != HM_OK) return rc;
        if (tok == eos_token) break;  // the reference leaves the loop without storing the token
        generated.push_back((uint32_t)tok);
        h_tokens[(*n_out)++] = tok;
        current = tok;
    }
    return finish_sync();
}

int HfModel::bench_decode(int64_t first_id, int n_steps, float *ms_out, int32_t *h_tokens) {
    if (!finalized_) return hm_set_error(ctx_, HM_ERR_STATE, "model not finalized");
    return with_whole_step_retry([&] { return bench_decode_once(first_id, n_steps, ms_out, h_tokens); });
}

int HfModel::bench_decode_once(int64_t first_id, int n_steps, float *ms_out, int32_t *h_tokens) {
    if (!finalized_) return hm_set_error(ctx_, HM_ERR_STATE, "model not finalized");
    if (n_steps <= 0 || n_steps > plan_->out_capacity())
        return hm_set_error(ctx_, HM_ERR_INVALID, "bench_decode: bad step count %d", n_steps);
    if (kv_cache_len() + n_steps > max_seq_len_)
        return hm_set_error(ctx_, HM_ERR_STATE, "KV cache full (%d + %d > %d)", kv_cache_len(), n_steps, max_seq_len_);
    std::vector<int32_t> ids;
    int rc = check_ids(&first_id, 1, ids);
    if (rc != HM_OK) return rc;
    if ((rc = plan_->arm(ids.data(), 1)) != HM_OK) return rc;
    std::vector<Buffer *> inputs;
    step_inputs(inputs);
    hipEvent_t e0, e1;
    HM_HIP(ctx_, hipEventCreate(&e0));
    HM_HIP(ctx_, hipEventCreate(&e1));
    HM_HIP(ctx_, hipEventRecord(e0, ctx_->stream));
    for (int i = 0; i < n_steps; i++)
        if ((rc = plan_->run_kv(inputs, weight_bufs_, max_seq_len_)) != HM_OK) break;
    if (rc == HM_OK) {
        HM_HIP(ctx_, hipEventRecord(e1, ctx_->stream));
        HM_HIP(ctx_, hipEventSynchronize(e1));
        HM_HIP(ctx_, hipEventElapsedTime(ms_out, e0, e1));
    }
    (void)hipEventDestroy(e0);
    (void)hipEventDestroy(e1);
    if (rc != HM_OK) return rc;
    if (h_tokens) rc = hm_download(ctx_, h_tokens, plan_->out_tokens(), (size_t)n_steps * 4);
    return rc == HM_OK ? finish_sync() : rc;
}

int HfModel::time_kernels(int rounds, std::vector<StepProfile> &out) {
    if (!finalized_) return hm_set_error(ctx_, HM_ERR_STATE, "model not finalized");
    int32_t tok = 0;
    int rc = plan_->arm(&tok, 1);
    if (rc != HM_OK) return rc;
    std::vector<Buffer *> inputs;
    step_inputs(inputs);
    return plan_->time_kernels(inputs, weight_bufs_, max_seq_len_, rounds, out);
}

int HfModel::profile_step(int64_t token_id, std::vector<StepProfile> &out) {
    if (!finalized_) return hm_set_error(ctx_, HM_ERR_STATE, "model not finalized");
    std::vector<int32_t> ids;
    int rc = check_ids(&token_id, 1, ids);
    if (rc != HM_OK) return rc;
    if ((rc = plan_->arm(ids.data(), 1)) != HM_OK) return rc;
    std::vector<Buffer *> inputs;
    step_inputs(inputs);
    return plan_->profile_step(inputs, weight_bufs_, max_seq_len_, out);
}

}  // namespace homura
