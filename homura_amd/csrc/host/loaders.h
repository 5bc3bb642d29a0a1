// Checkpoint containers read straight into the GPU model: GGUF (reference src/gguf.rs), HF
// safetensors + config.json (reference src/hf/safetensors.rs, src/hf/config.rs, the loading
// half of src/hf/weights.rs and src/hf/model.rs:75-146). Files are memory-mapped; tensors go
// from the mapping to HBM in the layout the kernels stream (no host-side transposes).
#pragma once

#include <cstdint>
#include <map>
#include <memory>
#include <string>
#include <vector>

#include "hf.h"
#include "json.h"

namespace homura {

// Read-only memory mapping of a whole file.
class MappedFile {
  public:
    MappedFile() = default;
    MappedFile(const MappedFile &) = delete;
    MappedFile &operator=(const MappedFile &) = delete;
    ~MappedFile();
    bool open(const std::string &path, std::string *err);
    const uint8_t *data() const { return data_; }
    size_t size() const { return size_; }

  private:
    const uint8_t *data_ = nullptr;
    size_t size_ = 0;
};

// ── GGUF ─────────────────────────────────────────────────────────────────────

// GGML tensor type codes (reference src/gguf.rs:25-57)
enum class GgmlType : uint32_t {
    F32 = 0, F16 = 1, Q4_0 = 2, Q4_1 = 3, Q5_0 = 6, Q5_1 = 7, Q8_0 = 8, Q8_1 = 9, Q2K = 10, Q3K = 11,
    Q4K = 12, Q5K = 13, Q6K = 14, Q8K = 15, IQ2XXS = 16, IQ2XS = 17, IQ3XXS = 18, IQ1S = 19, IQ4NL = 20,
    IQ3S = 21, IQ2S = 22, IQ4XS = 23, I8 = 24, I16 = 25, I32 = 26, I64 = 27, F64 = 28, IQ1M = 29, BF16 = 30,
};
bool ggml_type_known(uint32_t code);
size_t ggml_block_size(GgmlType t);  // elements per block (reference src/gguf.rs:115-132)
size_t ggml_type_size(GgmlType t);   // bytes per block (reference src/gguf.rs:135-164)
const char *ggml_type_name(GgmlType t);

// GGUF metadata value (reference GgufValue, src/gguf.rs:184-199)
struct GgufValue {
    enum Kind { U8, I8, U16, I16, U32, I32, F32, Bool, String, Array, U64, I64, F64 } kind = U8;
    uint64_t u = 0;  // unsigned kinds and Bool
    int64_t i = 0;   // signed kinds
    double f = 0;    // F32, F64
    std::string s;
    std::vector<GgufValue> arr;
    // the reference's lenient accessors (src/gguf.rs:200-233)
    bool as_u64(uint64_t *out) const;
    bool as_u32(uint32_t *out) const;
    bool as_f32(float *out) const;
    bool as_str(std::string *out) const;
};

struct GgufTensorInfo {
    std::string name;
    std::vector<uint64_t> shape;  // outermost first (the file stores innermost first)
    GgmlType type = GgmlType::F32;
    uint64_t offset = 0;  // inside the aligned data region
    uint64_t num_elements() const;
    size_t byte_size() const;
};

class GgufFile {
  public:
    // reference GgufFile::load (src/gguf.rs:345-451); nullptr + *err on failure
    static std::unique_ptr<GgufFile> load(const std::string &path, std::string *err);

    uint32_t version() const { return version_; }
    const std::vector<GgufTensorInfo> &tensors() const { return tensors_; }
    const std::map<std::string, GgufValue> &metadata() const { return metadata_; }
    const GgufTensorInfo *tensor_info(const std::string &name) const;
    const uint8_t *tensor_data(const GgufTensorInfo &info) const;  // raw bytes, no dequantisation
    const GgufValue *meta(const std::string &key) const;
    bool architecture(std::string *out) const;
    size_t data_offset() const { return data_offset_; }
    // reference GgufFile::transformer_config (src/gguf.rs:508-582)
    bool transformer_config(TransformerConfig *cfg, std::string *err) const;

  private:
    GgufFile() = default;
    MappedFile file_;
    uint32_t version_ = 0;
    size_t data_offset_ = 0;
    std::map<std::string, GgufValue> metadata_;
    std::vector<GgufTensorInfo> tensors_;
    std::map<std::string, size_t> by_name_;
};

// reference GgufFile::load_f32_buffer (src/gguf.rs:727-776): n elements of a GGML type as f32
bool ggml_to_f32(GgmlType type, const uint8_t *src, size_t n, std::vector<float> *out, std::string *err);

// reference load_transformer_weights + HfModel::load for a GGUF file (src/gguf.rs:589-708): projection
// weights stay the raw blocks (Q8_0, Q4_0) or become bf16 (F32/F16/BF16 files); norms, biases and the
// embedding become f32; the LM head is f32 in the quantised plan. Returns nullptr and sets the
// context error on failure.
std::unique_ptr<HfModel> load_gguf_model(hm_ctx *ctx, const std::string &path, int max_seq_len);

// ── safetensors + config.json ───────────────────────────────────────────────

struct SafeTensorInfo {
    std::string name, dtype;  // "BF16", "F16", "F32", ...
    std::vector<uint64_t> shape;
    size_t begin = 0, end = 0;  // byte range inside the data region
};

class SafeTensorsFile {
  public:
    // reference load_safetensors_impl (src/hf/safetensors.rs:38-99), without the conversions
    static std::unique_ptr<SafeTensorsFile> load(const std::string &path, std::string *err);
    const std::vector<SafeTensorInfo> &tensors() const { return tensors_; }
    const SafeTensorInfo *find(const std::string &name) const;
    const uint8_t *data(const SafeTensorInfo &t) const { return file_.data() + data_base_ + t.begin; }

  private:
    SafeTensorsFile() = default;
    MappedFile file_;
    size_t data_base_ = 0;
    std::vector<SafeTensorInfo> tensors_;
    std::map<std::string, size_t> by_name_;
};

// reference TransformerConfig::load (src/hf/config.rs:49-54) with its serde defaults
bool transformer_config_from_json(const std::string &json_text, TransformerConfig *cfg, std::string *err);

// reference HfModel::load (src/hf/model.rs:75-146) + load_transformer_weights (src/hf/weights.rs:267-417):
// a directory with config.json and model.safetensors or model.safetensors.index.json + shards.
// Projections and LM head are used in bf16 (BF16 tensors as they are, F32 truncated to the top 16
// bits as the reference's f32_buf_to_bf16 does, F16 through f32).
std::unique_ptr<HfModel> load_hf_model_dir(hm_ctx *ctx, const std::string &dir, int max_seq_len);

}  // namespace homura
