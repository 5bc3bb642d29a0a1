// Host runtime that keeps the reference's names and call shapes (reference src/runtime.rs):
// Buffer, KvCache, SlotDesc, KernelStep, NativeOp, KvPlanInfo, ExecutionPlan. What differs is
// where the bytes live (HBM) and what a "compiled kernel" is (a launcher of prebuilt gfx950
// kernels instead of a dlsym'ed CPU function).
#pragma once

#include <cstdint>
#include <functional>
#include <memory>
#include <string>
#include <vector>

#include "../hm_common.h"

namespace homura {

enum class DType : int { F32 = HM_DTYPE_F32, BF16 = HM_DTYPE_BF16, Q8_0 = HM_DTYPE_Q8_0,
                         Q4_0 = HM_DTYPE_Q4_0, I64 = HM_DTYPE_I64, Q4_K = HM_DTYPE_Q4_K, Q6_K = HM_DTYPE_Q6_K };

// reference src/dtype.rs:8-92 (sizes and block maths of the supported subset)
size_t dtype_size_bytes(DType t);       // 0 for block types
bool dtype_is_quantized(DType t);
size_t dtype_block_size(DType t);       // elements per block (1 for plain types)
size_t dtype_block_bytes(DType t);
// bytes for n elements; returns 0 and sets *ok=false when n is not a multiple of the block
size_t dtype_bytes_for_elements(DType t, size_t n, bool *ok);

constexpr int64_t DIM_DYNAMIC = -1;  // reference src/shape.rs DIM_DYNAMIC

// A tensor in HBM: either owns its allocation or is a view into another Buffer / the KV
// cache (reference Buffer with BufferData::Owned / ::View, src/runtime.rs:35-299).
class Buffer {
  public:
    Buffer() = default;
    Buffer(const Buffer &) = delete;
    Buffer &operator=(const Buffer &) = delete;
    Buffer(Buffer &&o) noexcept;
    Buffer &operator=(Buffer &&o) noexcept;
    ~Buffer();

    // Allocates; returns an empty Buffer (ptr()==nullptr) and sets the ctx error on failure.
    static Buffer alloc(hm_ctx *ctx, const std::vector<int64_t> &shape, DType dtype);
    static Buffer alloc_bytes(hm_ctx *ctx, size_t bytes, const std::vector<int64_t> &shape, DType dtype);
    static Buffer view(void *ptr, size_t bytes, const std::vector<int64_t> &shape,
                       const std::vector<int64_t> &strides, DType dtype);

    void *ptr() const { return ptr_; }
    template <typename T> T *as() const { return reinterpret_cast<T *>(ptr_); }
    size_t bytes() const { return bytes_; }
    const std::vector<int64_t> &shape() const { return shape_; }
    const std::vector<int64_t> &strides() const { return strides_; }
    DType dtype() const { return dtype_; }
    bool is_view() const { return !owned_; }
    explicit operator bool() const { return ptr_ != nullptr; }

  private:
    void release();
    hm_ctx *ctx_ = nullptr;
    void *ptr_ = nullptr;
    size_t bytes_ = 0;
    std::vector<int64_t> shape_, strides_;
    DType dtype_ = DType::F32;
    bool owned_ = false;
};

std::vector<int64_t> row_major_strides(const std::vector<int64_t> &shape);

// Persistent KV cache (reference KvCache, src/runtime.rs:355-650): per layer two buffers
// [1][heads][max_len][head_dim], zero-filled, here bf16 in HBM (the reference keeps f32 in
// host memory). append_* writes new rows at current_len, view_* exposes
// [0, current_len + new_tokens) with max_len strides, advance_by commits.
class KvCache {
  public:
    static std::unique_ptr<KvCache> create(hm_ctx *ctx, int num_layers, int num_heads, int max_len,
                                           int head_dim);
    // new_k / new_v: f32 [1][heads][new_seq][head_dim] in HBM. HM_ERR_STATE when full.
    int append_key(int layer, const Buffer &new_k);
    int append_value(int layer, const Buffer &new_v);
    // Bookkeeping half of an append whose rows a fused kernel has already written.
    int note_appended(int new_seq);
    Buffer view_key(int layer) const;
    Buffer view_value(int layer) const;
    void advance_by(int n) { current_len_ += n; new_tokens_ = 0; }
    void reset(int initial_len) { current_len_ = initial_len; new_tokens_ = 0; }
    int current_len() const { return current_len_; }
    int new_tokens() const { return new_tokens_; }
    int max_len() const { return max_len_; }
    int num_heads() const { return num_heads_; }
    int head_dim() const { return head_dim_; }
    int num_layers() const { return (int)key_.size(); }
    uint16_t *key_ptr(int layer) const { return key_[layer].as<uint16_t>(); }
    uint16_t *value_ptr(int layer) const { return value_[layer].as<uint16_t>(); }
    // Bulk load of prefill rows (reference ExecutionPlan::init_kv_cache, src/runtime.rs:1898-1938):
    // host f32 [1][heads][seq_len][head_dim] -> bf16 rows [0, seq_len).
    int load_from_host(int layer, const float *h_k, const float *h_v, int seq_len);

  private:
    Buffer view_single(const Buffer &src, int seq_len) const;
    int append_into(Buffer &dst_k_or_v, const Buffer &src, bool is_value, int layer);
    hm_ctx *ctx_ = nullptr;
    std::vector<Buffer> key_, value_;
    int current_len_ = 0, new_tokens_ = 0, max_len_ = 0, num_heads_ = 0, head_dim_ = 0;
};

// reference SlotDesc / KernelStep / NativeOp / KvPlanInfo (src/runtime.rs:1044-1105)
struct SlotDesc {
    std::vector<int64_t> shape;  // DIM_DYNAMIC for seq-dependent dims
    DType dtype;
    std::string name;            // for diagnostics and the weight-slot listing
};

enum class NativeOpKind { None, Concat };
struct NativeOp {
    NativeOpKind kind = NativeOpKind::None;
    int axis = 0;
};

struct KernelStep {
    static constexpr size_t NATIVE = (size_t)-1;
    size_t kernel_idx = NATIVE;
    std::vector<size_t> input_slots;
    std::vector<size_t> output_slots;
    NativeOp native_op;
    static KernelStep kernel(size_t idx, std::vector<size_t> in, std::vector<size_t> out) {
        KernelStep s;
        s.kernel_idx = idx;
        s.input_slots = std::move(in);
        s.output_slots = std::move(out);
        return s;
    }
};

struct KvPlanInfo {
    int num_layers = 0, num_heads = 0, head_dim = 0;
    std::vector<size_t> past_kv_input_slots;      // [l0_k, l0_v, l1_k, ...]
    std::vector<size_t> present_kv_output_slots;  // same order
};

class ExecutionPlan;

// What CompiledGraph is in the reference (src/runtime.rs:710-1038): the callable behind one
// kernel index. Here: a label plus a launcher that enqueues prebuilt HIP kernels.
struct StepContext {
    hm_ctx *ctx;
    ExecutionPlan *plan;
    const std::vector<Buffer *> &pool;  // slot -> buffer (inputs, weights, intermediates)
    const KernelStep &step;
    bool timing = false;  // launched over and over to be timed: a launch that would end the step must not move the cursor
};
// One HIP kernel launch inside a compiled kernel, named so that timings and byte counts can be
// reported per device kernel.
struct DeviceLaunch {
    std::string name;                 // e.g. "gemv_bf16[qkv]", "gqa_decode_attn"
    double bytes_fixed = 0;           // algorithmic bytes per launch (weights + activations)
    double bytes_per_kv_row = 0;      // plus this much per cached row (attention)
    bool moves_cursor = false;        // advances the DecodeState (must run exactly once per step)
    int hip_launches = 1;             // HIP kernels this entry enqueues
    // A plan may carry two ways through the layers: one launch per projection, or one launch for the
    // whole step. Entries of the way that is switched off are skipped.
    enum class Mode { Always, PerKernel, WholeStep };
    Mode mode = Mode::Always;
    std::function<int(const StepContext &)> fn;
};
struct CompiledKernel {
    std::string ops_label;  // "Embed", "QKV+QKNorm+RoPE", "Attn", "MLP", "LMHead", "QuantMM[q]", ...
    std::vector<DeviceLaunch> launches;
    int launch(const StepContext &sc, bool whole_step) const {
        for (const auto &l : launches) {
            if (l.mode == (whole_step ? DeviceLaunch::Mode::PerKernel : DeviceLaunch::Mode::WholeStep)) continue;
            int rc = l.fn(sc);
            if (rc != HM_OK) return rc;
        }
        return HM_OK;
    }
};

struct StepProfile {
    std::string label;  // device kernel name
    float ms = 0;       // summed over the launches
    int launches = 0;
    double bytes = 0;   // algorithmic bytes summed over the launches
};

// Ordered kernel dispatch with slot routing (reference ExecutionPlan, src/runtime.rs:1113-1951).
// The plan is static for seq == 1: every intermediate slot is allocated once at construction
// (the reference re-resolves symbolic shapes and rebuilds a buffer pool per call,
// src/runtime.rs:1684-1692); the position comes from a device-resident DecodeState so the
// whole step can be replayed from one captured HIP graph.
class ExecutionPlan {
  public:
    ExecutionPlan(hm_ctx *ctx, std::vector<CompiledKernel> kernels, std::vector<KernelStep> steps,
                  size_t num_slots, std::vector<size_t> input_slots,
                  std::vector<size_t> weight_slots, std::vector<size_t> output_slots,
                  std::vector<SlotDesc> slot_descs);
    ~ExecutionPlan();

    void set_kv_info(KvPlanInfo info) { kv_info_ = std::move(info); has_kv_info_ = true; }
    // Make `slot` a view into `base_slot`'s allocation at `byte_offset` (the base is grown to
    // hold it). Lets one kernel fill several adjacent slots (q|k|v) in a single pass.
    void alias_slot(size_t slot, size_t base_slot, size_t byte_offset);
    // Allocate the intermediates (seq = 1) and the decode cursor. Call once.
    int prepare(int max_out_tokens);

    // One decode step on top of the internal KvCache (reference run_kv,
    // src/runtime.rs:1580-1892). `inputs` are the non-KV model inputs in input_slots order
    // (input_ids, mask, cos, sin); `weights` in weight_slots order. Creates the cache on first
    // use with `max_seq_len` rows. The step's logits land in the logits slot; the greedy pick is
    // appended to the device token list. HM_ERR_STATE when the cache is full.
    int run_kv(const std::vector<Buffer *> &inputs, std::vector<Buffer> &weights, int max_seq_len);

    int init_kv_cache(const float *const *h_kv, int seq_len, int max_seq_len);
    void reset_kv_cache();
    int kv_cache_len() const { return kv_cache_ ? kv_cache_->current_len() : 0; }
    KvCache *kv_cache() { return kv_cache_.get(); }
    int ensure_kv_cache(int max_seq_len);

    // decode cursor (device) and the lists around it
    DecodeState *state() const { return state_.as<DecodeState>(); }
    int32_t *forced_ids() const { return forced_.as<int32_t>(); }
    int32_t *out_tokens() const { return out_tokens_.as<int32_t>(); }
    int out_capacity() const { return out_cap_; }
    // Arm the cursor: pos = cache length, step = 0, the given ids forced for the first steps.
    int arm(const int32_t *h_forced, int n_forced);

    // Graph replay of the step (captured lazily on first use; arguments never change).
    int enable_graph(bool on);
    bool graph_enabled() const { return use_graph_; }
    // Take the whole-step launch (when the plan has one) instead of the per-projection launches.
    int set_whole_step(bool on);
    bool whole_step() const { return whole_step_; }
    // Forget the recorded step (its launches' arguments or kernels are about to change); the next run records anew.
    int invalidate_graph();
    bool skips(const DeviceLaunch &l) const {
        return l.mode == (whole_step_ ? DeviceLaunch::Mode::PerKernel : DeviceLaunch::Mode::WholeStep);
    }
    // Called before a step is enqueued or captured, with the KV cache in place (device tables that
    // depend on the cache's addresses are refreshed here, outside any capture).
    void set_pre_run(std::function<int()> fn) { pre_run_ = std::move(fn); }
    // Rows the decode attention's grid covers in a recorded step (0: the cache's capacity). Whoever sets it keeps
    // the live rows within it and drops the recorded step when it changes.
    int attn_span() const { return attn_span_; }
    void set_attn_span(int rows) { attn_span_ = rows; }

    // Per-kernel timing of one step (HOMURA_PROFILE analogue, reference src/runtime.rs:1849-1873):
    // HIP events around every device launch of a real decode step.
    int profile_step(const std::vector<Buffer *> &inputs, std::vector<Buffer> &weights,
                     int max_seq_len, std::vector<StepProfile> &out);
    // Kernel-by-kernel timing for roofline figures: for every device-kernel name, all its
    // launches of the step (one per layer, i.e. different weights each time, so nothing is
    // cache-resident) are issued back to back `rounds` times between two HIP events. Launches
    // that move the cursor are skipped. Leaves activations and the current cache row in an
    // unspecified state: call when the decode is over.
    int time_kernels(const std::vector<Buffer *> &inputs, std::vector<Buffer> &weights,
                     int max_seq_len, int rounds, std::vector<StepProfile> &out);

    const std::vector<KernelStep> &steps() const { return steps_; }
    const std::vector<CompiledKernel> &kernels() const { return kernels_; }
    const std::vector<SlotDesc> &slot_descs() const { return slot_descs_; }
    const std::vector<size_t> &input_slots() const { return input_slots_; }
    const std::vector<size_t> &weight_slots() const { return weight_slots_; }
    const std::vector<size_t> &output_slots() const { return output_slots_; }
    size_t num_slots() const { return num_slots_; }
    Buffer *slot(size_t s) { return pool_[s]; }
    hm_ctx *ctx() const { return ctx_; }
    int launches_per_step() const;

  private:
    int bind(const std::vector<Buffer *> &inputs, std::vector<Buffer> &weights);
    int run_steps(std::vector<StepProfile> *profile);
    hm_ctx *ctx_;
    std::vector<CompiledKernel> kernels_;
    std::vector<KernelStep> steps_;
    size_t num_slots_;
    std::vector<size_t> input_slots_, weight_slots_, output_slots_;
    std::vector<SlotDesc> slot_descs_;
    KvPlanInfo kv_info_;
    bool has_kv_info_ = false;
    std::unique_ptr<KvCache> kv_cache_;
    struct Alias { size_t slot, base, offset; };
    std::vector<Alias> aliases_;
    std::vector<Buffer> owned_;     // intermediates
    std::vector<Buffer> kv_views_;  // per-step views of the cache bound to present_kv slots
    std::vector<Buffer *> pool_;
    Buffer state_, forced_, out_tokens_;
    // arm(): the cursor and the forced ids go out from pinned host memory with asynchronous copies (no stream
    // synchronisation per call); the event tells when that memory may be written again
    void *arm_pinned_ = nullptr;
    hipEvent_t arm_done_ = nullptr;
    int out_cap_ = 0;
    bool prepared_ = false;
    bool use_graph_ = false;
    bool whole_step_ = false;
    std::function<int()> pre_run_;
    int attn_span_ = 0;
    hipGraph_t graph_ = nullptr;
    hipGraphExec_t graph_exec_ = nullptr;
};

}  // namespace homura
