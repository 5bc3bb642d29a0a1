// Buffer, KvCache and ExecutionPlan on HBM (see runtime.h).
#include "runtime.h"

#include <algorithm>
#include <map>

namespace homura {

// ── dtype maths (reference src/dtype.rs:8-92) ────────────────────────────────

size_t dtype_size_bytes(DType t) {
    switch (t) {
    case DType::F32: return 4;
    case DType::BF16: return 2;
    case DType::I64: return 8;
    default: return 0;
    }
}
bool dtype_is_quantized(DType t) {
    return t == DType::Q8_0 || t == DType::Q4_0 || t == DType::Q4_K || t == DType::Q6_K;
}
size_t dtype_block_size(DType t) {
    if (t == DType::Q4_K || t == DType::Q6_K) return 256;
    return dtype_is_quantized(t) ? 32 : 1;
}
size_t dtype_block_bytes(DType t) {
    switch (t) {
    case DType::Q8_0: return 34;
    case DType::Q4_0: return 18;
    case DType::Q4_K: return 144;
    case DType::Q6_K: return 210;
    default: return dtype_size_bytes(t);
    }
}
size_t dtype_bytes_for_elements(DType t, size_t n, bool *ok) {
    if (ok) *ok = true;
    if (!dtype_is_quantized(t)) return n * dtype_size_bytes(t);
    if (n % dtype_block_size(t) != 0) {  // the reference panics "must be a multiple of block_size"
        if (ok) *ok = false;
        return 0;
    }
    return n / dtype_block_size(t) * dtype_block_bytes(t);
}

std::vector<int64_t> row_major_strides(const std::vector<int64_t> &shape) {
    std::vector<int64_t> st(shape.size(), 1);
    for (int i = (int)shape.size() - 2; i >= 0; i--) st[i] = st[i + 1] * shape[i + 1];
    return st;
}

// ── Buffer ───────────────────────────────────────────────────────────────────

Buffer::Buffer(Buffer &&o) noexcept { *this = std::move(o); }
Buffer &Buffer::operator=(Buffer &&o) noexcept {
    if (this != &o) {
        release();
        ctx_ = o.ctx_;
        ptr_ = o.ptr_;
        bytes_ = o.bytes_;
        shape_ = std::move(o.shape_);
        strides_ = std::move(o.strides_);
        dtype_ = o.dtype_;
        owned_ = o.owned_;
        o.ptr_ = nullptr;
        o.owned_ = false;
        o.bytes_ = 0;
    }
    return *this;
}
Buffer::~Buffer() { release(); }
void Buffer::release() {
    if (owned_ && ptr_ && ctx_) hm_free(ctx_, ptr_);
    ptr_ = nullptr;
    owned_ = false;
}

Buffer Buffer::alloc_bytes(hm_ctx *ctx, size_t bytes, const std::vector<int64_t> &shape,
                           DType dtype) {
    Buffer b;
    void *p = nullptr;
    if (hm_alloc(ctx, bytes, &p) != HM_OK) return b;
    b.ctx_ = ctx;
    b.ptr_ = p;
    b.bytes_ = bytes;
    b.shape_ = shape;
    b.strides_ = row_major_strides(shape);
    b.dtype_ = dtype;
    b.owned_ = true;
    return b;
}

Buffer Buffer::alloc(hm_ctx *ctx, const std::vector<int64_t> &shape, DType dtype) {
    size_t n = 1;
    for (auto d : shape) n *= (size_t)(d < 0 ? 1 : d);
    bool ok = true;
    size_t bytes = dtype_bytes_for_elements(dtype, n, &ok);
    if (!ok) {
        hm_set_error(ctx, HM_ERR_INVALID, "element count %zu is not a multiple of the block size", n);
        return Buffer();
    }
    return alloc_bytes(ctx, bytes, shape, dtype);
}

Buffer Buffer::view(void *ptr, size_t bytes, const std::vector<int64_t> &shape,
                    const std::vector<int64_t> &strides, DType dtype) {
    Buffer b;
    b.ptr_ = ptr;
    b.bytes_ = bytes;
    b.shape_ = shape;
    b.strides_ = strides;
    b.dtype_ = dtype;
    b.owned_ = false;
    return b;
}

// ── KvCache ──────────────────────────────────────────────────────────────────

std::unique_ptr<KvCache> KvCache::create(hm_ctx *ctx, int num_layers, int num_heads, int max_len,
                                         int head_dim) {
    std::unique_ptr<KvCache> c(new KvCache());
    c->ctx_ = ctx;
    c->max_len_ = max_len;
    c->num_heads_ = num_heads;
    c->head_dim_ = head_dim;
    const std::vector<int64_t> shape{1, num_heads, max_len, head_dim};
    for (int l = 0; l < num_layers; l++) {
        Buffer k = Buffer::alloc(ctx, shape, DType::BF16);
        Buffer v = Buffer::alloc(ctx, shape, DType::BF16);
        if (!k || !v) return nullptr;
        // zero-initialised like the reference (src/runtime.rs:399-406)
        if (hm_fill_zero(ctx, k.ptr(), k.bytes()) != HM_OK || hm_fill_zero(ctx, v.ptr(), v.bytes()) != HM_OK)
            return nullptr;
        c->key_.push_back(std::move(k));
        c->value_.push_back(std::move(v));
    }
    return c;
}

int KvCache::note_appended(int new_seq) {
    if (current_len_ + new_seq > max_len_)
        return hm_set_error(ctx_, HM_ERR_STATE, "KV cache full (%d + %d > %d)", current_len_, new_seq, max_len_);
    new_tokens_ = new_seq;
    return HM_OK;
}

int KvCache::append_key(int layer, const Buffer &new_k) {
    const int new_seq = (int)new_k.shape()[2];
    int rc = note_appended(new_seq);
    if (rc != HM_OK) return rc;
    // K and V go through the same row writer; the value side is given a throw-away target of the
    // same row so that a key-only append stays a single launch.
    return hm_kv_append(ctx_, key_ptr(layer), key_ptr(layer), new_k.as<float>(), new_k.as<float>(), 1,
                        num_heads_, head_dim_, max_len_, current_len_, new_seq);
}

int KvCache::append_value(int layer, const Buffer &new_v) {
    const int new_seq = (int)new_v.shape()[2];
    int rc = note_appended(new_seq);
    if (rc != HM_OK) return rc;
    return hm_kv_append(ctx_, value_ptr(layer), value_ptr(layer), new_v.as<float>(), new_v.as<float>(),
                        1, num_heads_, head_dim_, max_len_, current_len_, new_seq);
}

Buffer KvCache::view_single(const Buffer &src, int seq_len) const {
    // shape [1][heads][seq_len][hd] with max_len-based strides (reference src/runtime.rs:600-625)
    return Buffer::view(src.ptr(), src.bytes(), {1, num_heads_, seq_len, head_dim_},
                        {(int64_t)num_heads_ * max_len_ * head_dim_, (int64_t)max_len_ * head_dim_,
                         head_dim_, 1},
                        DType::BF16);
}
Buffer KvCache::view_key(int layer) const { return view_single(key_[layer], current_len_ + new_tokens_); }
Buffer KvCache::view_value(int layer) const { return view_single(value_[layer], current_len_ + new_tokens_); }

int KvCache::load_from_host(int layer, const float *h_k, const float *h_v, int seq_len) {
    if (seq_len > max_len_)
        return hm_set_error(ctx_, HM_ERR_STATE, "KV cache full (0 + %d > %d)", seq_len, max_len_);
    if (seq_len == 0) return HM_OK;
    const size_t n = (size_t)num_heads_ * seq_len * head_dim_;
    Buffer sk = Buffer::alloc(ctx_, {1, num_heads_, seq_len, head_dim_}, DType::F32);
    Buffer sv = Buffer::alloc(ctx_, {1, num_heads_, seq_len, head_dim_}, DType::F32);
    if (!sk || !sv) return HM_ERR_OOM;
    int rc;
    if ((rc = hm_upload(ctx_, sk.ptr(), h_k, n * 4)) != HM_OK) return rc;
    if ((rc = hm_upload(ctx_, sv.ptr(), h_v, n * 4)) != HM_OK) return rc;
    rc = hm_kv_append(ctx_, key_ptr(layer), value_ptr(layer), sk.as<float>(), sv.as<float>(), 1,
                      num_heads_, head_dim_, max_len_, 0, seq_len);
    if (rc != HM_OK) return rc;
    return hm_sync(ctx_);
}

// ── ExecutionPlan ────────────────────────────────────────────────────────────

ExecutionPlan::ExecutionPlan(hm_ctx *ctx, std::vector<CompiledKernel> kernels,
                             std::vector<KernelStep> steps, size_t num_slots,
                             std::vector<size_t> input_slots, std::vector<size_t> weight_slots,
                             std::vector<size_t> output_slots, std::vector<SlotDesc> slot_descs)
    : ctx_(ctx), kernels_(std::move(kernels)), steps_(std::move(steps)), num_slots_(num_slots),
      input_slots_(std::move(input_slots)), weight_slots_(std::move(weight_slots)),
      output_slots_(std::move(output_slots)), slot_descs_(std::move(slot_descs)) {
    pool_.assign(num_slots_, nullptr);
}

ExecutionPlan::~ExecutionPlan() {
    if (arm_done_) {
        (void)hipEventSynchronize(arm_done_);
        (void)hipEventDestroy(arm_done_);
    }
    if (arm_pinned_) (void)hipHostFree(arm_pinned_);
    if (graph_exec_) (void)hipGraphExecDestroy(graph_exec_);
    if (graph_) (void)hipGraphDestroy(graph_);
}

void ExecutionPlan::alias_slot(size_t slot, size_t base_slot, size_t byte_offset) {
    aliases_.push_back(Alias{slot, base_slot, byte_offset});
}

static size_t slot_bytes(const SlotDesc &d) {
    size_t n = 1;
    for (auto v : d.shape) n *= (size_t)(v == DIM_DYNAMIC ? 1 : v);
    return dtype_bytes_for_elements(d.dtype, n, nullptr);
}

int ExecutionPlan::prepare(int max_out_tokens) {
    if (prepared_) return HM_OK;
    std::vector<bool> external(num_slots_, false);
    std::vector<size_t> extra(num_slots_, 0);
    for (auto &a : aliases_) {
        external[a.slot] = true;  // not allocated on its own
        extra[a.base] = std::max(extra[a.base], a.offset + slot_bytes(slot_descs_[a.slot]));
    }
    for (auto s : input_slots_) external[s] = true;
    for (auto s : weight_slots_) external[s] = true;
    if (has_kv_info_) {
        for (auto s : kv_info_.past_kv_input_slots) external[s] = true;
        for (auto s : kv_info_.present_kv_output_slots) external[s] = true;
    }
    owned_.reserve(num_slots_ + aliases_.size());
    for (size_t s = 0; s < num_slots_; s++) {
        if (external[s]) continue;
        std::vector<int64_t> shape = slot_descs_[s].shape;
        for (auto &d : shape)
            if (d == DIM_DYNAMIC) d = 1;  // the plan is specialised to one new token per step
        const size_t bytes = std::max(slot_bytes(slot_descs_[s]), extra[s]);
        Buffer b = Buffer::alloc_bytes(ctx_, bytes, shape, slot_descs_[s].dtype);
        if (!b) return HM_ERR_OOM;
        owned_.push_back(std::move(b));
        pool_[s] = &owned_.back();
    }
    owned_.reserve(owned_.size() + aliases_.size());
    for (auto &a : aliases_) {
        if (!pool_[a.base]) return hm_set_error(ctx_, HM_ERR_STATE, "alias base slot %zu is not an intermediate", a.base);
        std::vector<int64_t> shape = slot_descs_[a.slot].shape;
        for (auto &d : shape)
            if (d == DIM_DYNAMIC) d = 1;
        owned_.push_back(Buffer::view((char *)pool_[a.base]->ptr() + a.offset,
                                      slot_bytes(slot_descs_[a.slot]), shape,
                                      row_major_strides(shape), slot_descs_[a.slot].dtype));
        pool_[a.slot] = &owned_.back();
    }
    out_cap_ = max_out_tokens;
    state_ = Buffer::alloc_bytes(ctx_, sizeof(DecodeState), {1}, DType::F32);
    forced_ = Buffer::alloc_bytes(ctx_, (size_t)max_out_tokens * 4, {max_out_tokens}, DType::F32);
    out_tokens_ = Buffer::alloc_bytes(ctx_, (size_t)max_out_tokens * 4, {max_out_tokens}, DType::F32);
    if (!state_ || !forced_ || !out_tokens_) return HM_ERR_OOM;
    int rc = hm_fill_zero(ctx_, state_.ptr(), sizeof(DecodeState));
    if (rc == HM_OK) rc = hm_fill_zero(ctx_, forced_.ptr(), forced_.bytes());
    if (rc == HM_OK) rc = hm_fill_zero(ctx_, out_tokens_.ptr(), out_tokens_.bytes());
    if (rc == HM_OK) rc = hm_sync(ctx_);
    prepared_ = rc == HM_OK;
    return rc;
}

int ExecutionPlan::ensure_kv_cache(int max_seq_len) {
    if (kv_cache_) return HM_OK;
    if (!has_kv_info_) return hm_set_error(ctx_, HM_ERR_STATE, "run_kv called but plan has no KV cache info");
    kv_cache_ = KvCache::create(ctx_, kv_info_.num_layers, kv_info_.num_heads, max_seq_len,
                                kv_info_.head_dim);
    if (!kv_cache_) return HM_ERR_OOM;
    // bind cache views to the past/present KV slots once: the pointers never move
    kv_views_.clear();
    kv_views_.reserve(kv_info_.present_kv_output_slots.size() * 2);
    for (size_t i = 0; i < kv_info_.present_kv_output_slots.size(); i++) {
        const int layer = (int)(i / 2);
        const bool is_value = (i % 2) == 1;
        kv_views_.push_back(is_value ? kv_cache_->view_value(layer) : kv_cache_->view_key(layer));
        pool_[kv_info_.present_kv_output_slots[i]] = &kv_views_.back();
        pool_[kv_info_.past_kv_input_slots[i]] = &kv_views_.back();
    }
    return HM_OK;
}

int ExecutionPlan::init_kv_cache(const float *const *h_kv, int seq_len, int max_seq_len) {
    if (!has_kv_info_) return hm_set_error(ctx_, HM_ERR_STATE, "init_kv_cache called but plan has no KV cache info");
    if (kv_cache_ && kv_cache_->max_len() != max_seq_len) {
        kv_cache_.reset();
        if (graph_exec_) {  // captured pointers are gone
            (void)hipGraphExecDestroy(graph_exec_);
            graph_exec_ = nullptr;
        }
        if (graph_) {
            (void)hipGraphDestroy(graph_);
            graph_ = nullptr;
        }
    }
    int rc = ensure_kv_cache(max_seq_len);
    if (rc != HM_OK) return rc;
    for (int l = 0; l < kv_info_.num_layers; l++) {
        rc = kv_cache_->load_from_host(l, h_kv[2 * l], h_kv[2 * l + 1], seq_len);
        if (rc != HM_OK) return rc;
    }
    kv_cache_->reset(seq_len);
    return HM_OK;
}

void ExecutionPlan::reset_kv_cache() {
    if (kv_cache_) kv_cache_->reset(0);
}

int ExecutionPlan::arm(const int32_t *h_forced, int n_forced) {
    if (!prepared_) return hm_set_error(ctx_, HM_ERR_STATE, "plan not prepared");
    if (n_forced > out_cap_) return hm_set_error(ctx_, HM_ERR_INVALID, "%d forced ids exceed the plan's capacity %d", n_forced, out_cap_);
    const DecodeState st{kv_cache_len(), 0, 0, n_forced};
    if (!arm_pinned_) {
        HM_HIP(ctx_, hipHostMalloc(&arm_pinned_, sizeof(DecodeState) + (size_t)out_cap_ * 4, hipHostMallocDefault));
        HM_HIP(ctx_, hipEventCreateWithFlags(&arm_done_, hipEventDisableTiming));
    } else {
        HM_HIP(ctx_, hipEventSynchronize(arm_done_));  // the previous call's copies have read the staging memory
    }
    char *stage = static_cast<char *>(arm_pinned_);
    std::memcpy(stage, &st, sizeof(st));
    if (n_forced > 0) std::memcpy(stage + sizeof(st), h_forced, (size_t)n_forced * 4);
    HM_HIP(ctx_, hipMemcpyAsync(state_.ptr(), stage, sizeof(st), hipMemcpyHostToDevice, ctx_->stream));
    if (n_forced > 0)
        HM_HIP(ctx_, hipMemcpyAsync(forced_.ptr(), stage + sizeof(st), (size_t)n_forced * 4, hipMemcpyHostToDevice, ctx_->stream));
    HM_HIP(ctx_, hipEventRecord(arm_done_, ctx_->stream));
    return HM_OK;
}

int ExecutionPlan::bind(const std::vector<Buffer *> &inputs, std::vector<Buffer> &weights) {
    std::vector<size_t> non_kv;
    for (auto s : input_slots_)
        if (std::find(kv_info_.past_kv_input_slots.begin(), kv_info_.past_kv_input_slots.end(), s) ==
            kv_info_.past_kv_input_slots.end())
            non_kv.push_back(s);
    if (inputs.size() != non_kv.size())  // reference asserts the same (src/runtime.rs:1648-1654)
        return hm_set_error(ctx_, HM_ERR_INVALID, "run_kv: expected %zu non-KV inputs, got %zu",
                            non_kv.size(), inputs.size());
    if (weights.size() != weight_slots_.size())
        return hm_set_error(ctx_, HM_ERR_INVALID, "run_kv: expected %zu weights, got %zu",
                            weight_slots_.size(), weights.size());
    for (size_t i = 0; i < non_kv.size(); i++) pool_[non_kv[i]] = inputs[i];
    for (size_t i = 0; i < weight_slots_.size(); i++) pool_[weight_slots_[i]] = &weights[i];
    return HM_OK;
}

int ExecutionPlan::launches_per_step() const {
    int n = 0;
    for (const auto &st : steps_)
        if (st.native_op.kind == NativeOpKind::None)
            for (const auto &l : kernels_[st.kernel_idx].launches)
                if (!skips(l)) n += l.hip_launches;
    return n;
}

int ExecutionPlan::run_steps(std::vector<StepProfile> *profile) {
    hipEvent_t e0 = nullptr, e1 = nullptr;
    if (profile) {
        HM_HIP(ctx_, hipEventCreate(&e0));
        HM_HIP(ctx_, hipEventCreate(&e1));
    }
    const int kv_rows = kv_cache_ ? kv_cache_->current_len() + kv_cache_->new_tokens() : 0;
    std::map<std::string, size_t> by_label;
    for (size_t step_idx = 0; step_idx < steps_.size(); step_idx++) {
        const KernelStep &step = steps_[step_idx];
        if (step.native_op.kind == NativeOpKind::Concat) {
            // KV concat interception (reference src/runtime.rs:1729-1755): the rows were written
            // into the cache by the QKV kernel's fused append; what remains is handing the
            // cache view to the consumer, which ensure_kv_cache() has bound for good.
            const size_t out_slot = step.output_slots[0];
            if (!pool_[out_slot])
                return hm_set_error(ctx_, HM_ERR_STATE, "buffer slot %zu not populated at step %zu", out_slot, step_idx);
            continue;
        }
        for (auto s : step.input_slots)
            if (!pool_[s])  // reference panics with the same message (src/runtime.rs:1700-1705)
                return hm_set_error(ctx_, HM_ERR_STATE, "buffer slot %zu not populated at step %zu", s, step_idx);
        const CompiledKernel &k = kernels_[step.kernel_idx];
        StepContext sc{ctx_, this, pool_, step};
        if (!profile) {
            int rc = k.launch(sc, whole_step_);
            if (rc != HM_OK) return rc;
            continue;
        }
        for (const DeviceLaunch &l : k.launches) {
            if (skips(l)) continue;
            HM_HIP(ctx_, hipEventRecord(e0, ctx_->stream));
            int rc = l.fn(sc);
            if (rc != HM_OK) return rc;
            HM_HIP(ctx_, hipEventRecord(e1, ctx_->stream));
            HM_HIP(ctx_, hipEventSynchronize(e1));
            float ms = 0;
            HM_HIP(ctx_, hipEventElapsedTime(&ms, e0, e1));
            auto it = by_label.find(l.name);
            if (it == by_label.end()) {
                by_label[l.name] = profile->size();
                profile->push_back(StepProfile{l.name, 0.f, 0, 0.0});
                it = by_label.find(l.name);
            }
            StepProfile &p = (*profile)[it->second];
            p.ms += ms;
            p.launches += 1;
            p.bytes += l.bytes_fixed + l.bytes_per_kv_row * kv_rows;
        }
    }
    if (profile) {
        (void)hipEventDestroy(e0);
        (void)hipEventDestroy(e1);
    }
    return HM_OK;
}

int ExecutionPlan::time_kernels(const std::vector<Buffer *> &inputs, std::vector<Buffer> &weights,
                                int max_seq_len, int rounds, std::vector<StepProfile> &out) {
    if (!prepared_) return hm_set_error(ctx_, HM_ERR_STATE, "plan not prepared");
    if (rounds < 1) return hm_set_error(ctx_, HM_ERR_INVALID, "time_kernels: rounds must be >= 1");
    int rc = ensure_kv_cache(max_seq_len);
    if (rc != HM_OK) return rc;
    if (kv_cache_->current_len() + 1 > kv_cache_->max_len())
        return hm_set_error(ctx_, HM_ERR_STATE, "KV cache full (%d + 1 > %d)", kv_cache_->current_len(), kv_cache_->max_len());
    if ((rc = bind(inputs, weights)) != HM_OK) return rc;
    if (pre_run_ && (rc = pre_run_()) != HM_OK) return rc;
    const int kv_rows = kv_cache_->current_len() + 1;
    std::vector<std::string> names;
    for (const auto &st : steps_) {
        if (st.native_op.kind != NativeOpKind::None) continue;
        for (const auto &l : kernels_[st.kernel_idx].launches)
            if (!l.moves_cursor && !skips(l) && std::find(names.begin(), names.end(), l.name) == names.end())
                names.push_back(l.name);
    }
    hipEvent_t e0, e1;
    HM_HIP(ctx_, hipEventCreate(&e0));
    HM_HIP(ctx_, hipEventCreate(&e1));
    for (const auto &name : names) {
        StepProfile p{name, 0.f, 0, 0.0};
        for (int r = -1; r < rounds; r++) {  // round -1 is an untimed warm-up
            if (r == 0) HM_HIP(ctx_, hipEventRecord(e0, ctx_->stream));
            for (const auto &st : steps_) {
                if (st.native_op.kind != NativeOpKind::None) continue;
                StepContext sc{ctx_, this, pool_, st, true};
                for (const auto &l : kernels_[st.kernel_idx].launches) {
                    if (l.name != name || skips(l)) continue;
                    if ((rc = l.fn(sc)) != HM_OK) return rc;
                    if (r >= 0) {
                        p.launches++;
                        p.bytes += l.bytes_fixed + l.bytes_per_kv_row * kv_rows;
                    }
                }
            }
        }
        HM_HIP(ctx_, hipEventRecord(e1, ctx_->stream));
        HM_HIP(ctx_, hipEventSynchronize(e1));
        HM_HIP(ctx_, hipEventElapsedTime(&p.ms, e0, e1));
        out.push_back(p);
    }
    (void)hipEventDestroy(e0);
    (void)hipEventDestroy(e1);
    return HM_OK;
}

int ExecutionPlan::enable_graph(bool on) {
    use_graph_ = on;
    return HM_OK;
}

int ExecutionPlan::set_whole_step(bool on) {
    if (on == whole_step_) return HM_OK;
    whole_step_ = on;
    return invalidate_graph();  // the captured step took the other way through the layers
}

int ExecutionPlan::invalidate_graph() {
    if (graph_exec_) {
        HM_HIP(ctx_, hipStreamSynchronize(ctx_->stream));
        (void)hipGraphExecDestroy(graph_exec_);
        graph_exec_ = nullptr;
    }
    if (graph_) {
        (void)hipGraphDestroy(graph_);
        graph_ = nullptr;
    }
    return HM_OK;
}

int ExecutionPlan::run_kv(const std::vector<Buffer *> &inputs, std::vector<Buffer> &weights,
                          int max_seq_len) {
    if (!prepared_) return hm_set_error(ctx_, HM_ERR_STATE, "plan not prepared");
    int rc = ensure_kv_cache(max_seq_len);
    if (rc != HM_OK) return rc;
    if ((rc = kv_cache_->note_appended(1)) != HM_OK) return rc;  // "KV cache full"
    if ((rc = bind(inputs, weights)) != HM_OK) return rc;
    if (pre_run_ && (rc = pre_run_()) != HM_OK) return rc;
    // A graph pays when a step is many launches. A step of one or two is quicker launched directly: the replay
    // of a one-node graph costs more on the GPU's queue than the kernel's own dispatch packet.
    if (use_graph_ && launches_per_step() > 2) {
        if (!graph_exec_) {
            if (graph_) {
                (void)hipGraphDestroy(graph_);
                graph_ = nullptr;
            }
            HM_HIP(ctx_, hipStreamBeginCapture(ctx_->stream, hipStreamCaptureModeRelaxed));
            rc = run_steps(nullptr);
            hipGraph_t g = nullptr;
            hipError_t e = hipStreamEndCapture(ctx_->stream, &g);
            if (rc != HM_OK) {
                if (g) (void)hipGraphDestroy(g);
                return rc;
            }
            HM_HIP(ctx_, e);
            graph_ = g;
            HM_HIP(ctx_, hipGraphInstantiate(&graph_exec_, graph_, nullptr, nullptr, 0));
        }
        HM_HIP(ctx_, hipGraphLaunch(graph_exec_, ctx_->stream));
    } else {
        rc = run_steps(nullptr);
        if (rc != HM_OK) return rc;
    }
    // one advance after all layers appended (reference src/runtime.rs:1875-1880)
    kv_cache_->advance_by(kv_cache_->new_tokens());
    return HM_OK;
}

int ExecutionPlan::profile_step(const std::vector<Buffer *> &inputs, std::vector<Buffer> &weights,
                                int max_seq_len, std::vector<StepProfile> &out) {
    if (!prepared_) return hm_set_error(ctx_, HM_ERR_STATE, "plan not prepared");
    int rc = ensure_kv_cache(max_seq_len);
    if (rc != HM_OK) return rc;
    if ((rc = kv_cache_->note_appended(1)) != HM_OK) return rc;
    if ((rc = bind(inputs, weights)) != HM_OK) return rc;
    if (pre_run_ && (rc = pre_run_()) != HM_OK) return rc;
    rc = run_steps(&out);
    if (rc != HM_OK) return rc;
    kv_cache_->advance_by(kv_cache_->new_tokens());
    return hm_sync(ctx_);
}

}  // namespace homura
