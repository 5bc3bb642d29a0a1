// GGUF, safetensors and config.json readers and the two model loaders built on them.
#include "loaders.h"

#include <fcntl.h>
#include <sys/mman.h>
#include <sys/stat.h>
#include <unistd.h>

#include <cerrno>
#include <cmath>
#include <cstdlib>
#include <cstring>
#include <set>

namespace homura {

// ── MappedFile ───────────────────────────────────────────────────────────────

MappedFile::~MappedFile() {
    if (data_ && size_) munmap(const_cast<uint8_t *>(data_), size_);
}

bool MappedFile::open(const std::string &path, std::string *err) {
    const int fd = ::open(path.c_str(), O_RDONLY);
    if (fd < 0) {
        *err = path + ": " + std::strerror(errno);
        return false;
    }
    struct stat st;
    if (fstat(fd, &st) != 0) {
        *err = path + ": " + std::strerror(errno);
        ::close(fd);
        return false;
    }
    size_ = (size_t)st.st_size;
    if (size_ == 0) {
        data_ = nullptr;
        ::close(fd);
        return true;
    }
    void *p = mmap(nullptr, size_, PROT_READ, MAP_PRIVATE, fd, 0);
    ::close(fd);
    if (p == MAP_FAILED) {
        *err = path + ": mmap failed: " + std::strerror(errno);
        size_ = 0;
        return false;
    }
    // reference: MADV_HUGEPAGE on the weight mapping (src/gguf.rs:351-360); here the pages are read
    // once, front to back, on their way to HBM
    madvise(p, size_, MADV_SEQUENTIAL);
    data_ = static_cast<const uint8_t *>(p);
    return true;
}

// ── scalar conversions (host) ────────────────────────────────────────────────

namespace {

// IEEE half bits -> f32, every pattern (reference f16_to_f32, src/gguf.rs:781-810)
float f16_bits_to_f32_host(uint16_t h) {
    const uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    const uint32_t exp = (h >> 10) & 0x1Fu;
    uint32_t man = h & 0x3FFu;
    uint32_t bits;
    if (exp == 0) {
        if (man == 0) {
            bits = sign;
        } else {  // subnormal: renormalise
            int e = -1;
            do {
                man <<= 1;
                e++;
            } while (!(man & 0x400u));
            bits = sign | ((uint32_t)(127 - 15 - e) << 23) | ((man & 0x3FFu) << 13);
        }
    } else if (exp == 31) {
        bits = sign | 0x7F800000u | (man << 13);
    } else {
        bits = sign | ((exp + 127 - 15) << 23) | (man << 13);
    }
    float f;
    std::memcpy(&f, &bits, 4);
    return f;
}

inline float bf16_bits_to_f32_host(uint16_t b) {
    const uint32_t bits = (uint32_t)b << 16;
    float f;
    std::memcpy(&f, &bits, 4);
    return f;
}

// top 16 bits (reference f32_buf_to_bf16, src/hf/weights.rs:206-214)
inline uint16_t f32_to_bf16_trunc_host(float f) {
    uint32_t bits;
    std::memcpy(&bits, &f, 4);
    return (uint16_t)(bits >> 16);
}

inline uint16_t rd16(const uint8_t *p) { return (uint16_t)(p[0] | (p[1] << 8)); }

// block dequantisation exactly as the GPU and the reference do it: one f32 multiply per weight
void dequant_q8_0_host(const uint8_t *src, float *dst, size_t n) {
    for (size_t b = 0; b < n / 32; b++) {
        const uint8_t *blk = src + b * 34;
        const float d = f16_bits_to_f32_host(rd16(blk));
        for (int j = 0; j < 32; j++) dst[b * 32 + j] = (float)(int8_t)blk[2 + j] * d;
    }
}
void dequant_q4_0_host(const uint8_t *src, float *dst, size_t n) {
    for (size_t b = 0; b < n / 32; b++) {
        const uint8_t *blk = src + b * 18;
        const float d = f16_bits_to_f32_host(rd16(blk));
        for (int j = 0; j < 16; j++) {
            dst[b * 32 + j] = (float)((blk[2 + j] & 0x0F) - 8) * d;
            dst[b * 32 + j + 16] = (float)((blk[2 + j] >> 4) - 8) * d;
        }
    }
}
// Q4_K (reference dequantize_q4_k, src/gguf.rs:835-882): weight e of a 256-wide super-block sits in
// sub-block s = e/32; sub-blocks 2p and 2p+1 share the 32 bytes at 16 + 32p (low and high nibbles);
// the 6-bit scale and minimum of sub-block s come out of the 12 bytes at offset 4.
// w = nibble * (d * scale) - dmin * minimum, three roundings, no fused multiply-add.
#pragma clang fp contract(off)
void dequant_q4_k_host(const uint8_t *src, float *dst, size_t n) {
    for (size_t b = 0; b < n / 256; b++) {
        const uint8_t *blk = src + b * 144, *pk = blk + 4;
        const float d = f16_bits_to_f32_host(rd16(blk)), dmin = f16_bits_to_f32_host(rd16(blk + 2));
        for (int s = 0; s < 8; s++) {
            int sc, mn;
            if (s < 4) {
                sc = pk[s] & 63;
                mn = pk[4 + s] & 63;
            } else {
                sc = (pk[4 + s] & 15) | ((pk[s - 4] >> 6) << 4);
                mn = (pk[4 + s] >> 4) | ((pk[s] >> 6) << 4);
            }
            const float scale = d * (float)sc;
            const float minimum = dmin * (float)mn;
            const uint8_t *q = blk + 16 + 32 * (s >> 1);
            float *o = dst + b * 256 + 32 * s;
            for (int l = 0; l < 32; l++) {
                const float prod = (float)((s & 1) ? (q[l] >> 4) : (q[l] & 15)) * scale;
                o[l] = prod - minimum;
            }
        }
    }
}
// Q6_K (reference dequantize_q6_k, src/gguf.rs:886-917): weight e = 128h + 32g + l has its low nibble in
// byte 64h + 32(g&1) + l (upper half of the byte for g >= 2), its two high bits at bit 2g of byte
// 128 + 32h + l, and the int8 scale 192 + 8h + 2g + l/16. w = (d * scale) * (q - 32).
void dequant_q6_k_host(const uint8_t *src, float *dst, size_t n) {
    for (size_t b = 0; b < n / 256; b++) {
        const uint8_t *blk = src + b * 210;
        const float d = f16_bits_to_f32_host(rd16(blk + 208));
        for (int e = 0; e < 256; e++) {
            const int h = e >> 7, g = (e & 127) >> 5, l = e & 31;
            const uint8_t lb = blk[64 * h + 32 * (g & 1) + l];
            const int lo = g >= 2 ? (lb >> 4) : (lb & 15);
            const int hi = (blk[128 + 32 * h + l] >> (2 * g)) & 3;
            const int q = (int)(int8_t)(lo | (hi << 4)) - 32;
            const float ds = d * (float)(int8_t)blk[192 + 8 * h + 2 * g + (l >> 4)];
            dst[b * 256 + e] = ds * (float)q;
        }
    }
}

}  // namespace

// ── GGML types ───────────────────────────────────────────────────────────────

bool ggml_type_known(uint32_t c) { return c <= 30 && c != 4 && c != 5; }

size_t ggml_block_size(GgmlType t) {
    switch (t) {
    case GgmlType::F32: case GgmlType::F64: case GgmlType::I8: case GgmlType::I16: case GgmlType::I32:
    case GgmlType::I64: case GgmlType::F16: case GgmlType::BF16:
        return 1;
    case GgmlType::Q4_0: case GgmlType::Q4_1: case GgmlType::Q5_0: case GgmlType::Q5_1: case GgmlType::Q8_0:
    case GgmlType::Q8_1:
        return 32;
    default:
        return 256;
    }
}

size_t ggml_type_size(GgmlType t) {
    switch (t) {
    case GgmlType::F32: return 4;
    case GgmlType::F64: return 8;
    case GgmlType::F16: case GgmlType::BF16: return 2;
    case GgmlType::I8: return 1;
    case GgmlType::I16: return 2;
    case GgmlType::I32: return 4;
    case GgmlType::I64: return 8;
    case GgmlType::Q4_0: return 18;
    case GgmlType::Q4_1: return 20;
    case GgmlType::Q5_0: return 22;
    case GgmlType::Q5_1: return 24;
    case GgmlType::Q8_0: return 34;
    case GgmlType::Q8_1: return 40;
    case GgmlType::Q2K: return 84;
    case GgmlType::Q3K: return 110;
    case GgmlType::Q4K: return 144;
    case GgmlType::Q5K: return 176;
    case GgmlType::Q6K: return 210;
    case GgmlType::Q8K: return 292;
    case GgmlType::IQ2XXS: return 66;
    case GgmlType::IQ2XS: return 74;
    case GgmlType::IQ3XXS: return 98;
    case GgmlType::IQ1S: return 50;
    case GgmlType::IQ4NL: return 18;
    case GgmlType::IQ3S: return 110;
    case GgmlType::IQ2S: return 82;
    case GgmlType::IQ4XS: return 36;
    case GgmlType::IQ1M: return 56;
    }
    return 0;
}

const char *ggml_type_name(GgmlType t) {
    switch (t) {
    case GgmlType::F32: return "F32";
    case GgmlType::F16: return "F16";
    case GgmlType::BF16: return "BF16";
    case GgmlType::F64: return "F64";
    case GgmlType::Q4_0: return "Q4_0";
    case GgmlType::Q4_1: return "Q4_1";
    case GgmlType::Q5_0: return "Q5_0";
    case GgmlType::Q5_1: return "Q5_1";
    case GgmlType::Q8_0: return "Q8_0";
    case GgmlType::Q8_1: return "Q8_1";
    case GgmlType::Q2K: return "Q2_K";
    case GgmlType::Q3K: return "Q3_K";
    case GgmlType::Q4K: return "Q4_K";
    case GgmlType::Q5K: return "Q5_K";
    case GgmlType::Q6K: return "Q6_K";
    case GgmlType::Q8K: return "Q8_K";
    case GgmlType::I8: return "I8";
    case GgmlType::I16: return "I16";
    case GgmlType::I32: return "I32";
    case GgmlType::I64: return "I64";
    default: return "IQ*";
    }
}

// ── GGUF values ──────────────────────────────────────────────────────────────

bool GgufValue::as_u64(uint64_t *out) const {
    switch (kind) {
    case U64: case U32: *out = u; return true;
    case I32: case I64: *out = (uint64_t)i; return true;
    default: return false;
    }
}
bool GgufValue::as_u32(uint32_t *out) const {
    switch (kind) {
    case U32: case U64: *out = (uint32_t)u; return true;
    case I32: *out = (uint32_t)i; return true;
    default: return false;
    }
}
bool GgufValue::as_f32(float *out) const {
    if (kind != F32 && kind != F64) return false;
    *out = (float)f;
    return true;
}
bool GgufValue::as_str(std::string *out) const {
    if (kind != String) return false;
    *out = s;
    return true;
}

uint64_t GgufTensorInfo::num_elements() const {
    uint64_t n = 1;
    for (uint64_t d : shape) n *= d;
    return n;
}
size_t GgufTensorInfo::byte_size() const {
    return (size_t)(num_elements() / ggml_block_size(type)) * ggml_type_size(type);
}

// ── GGUF parser ──────────────────────────────────────────────────────────────

namespace {

constexpr uint32_t GGUF_MAGIC = 0x46554747u;  // "GGUF", little-endian
constexpr size_t GGUF_DEFAULT_ALIGNMENT = 32;

struct Cursor {
    const uint8_t *p;
    size_t size, pos = 0;
    std::string err;
    bool need(size_t n) {
        if (n > size - pos) {  // pos <= size always
            err = "unexpected end of GGUF data at offset " + std::to_string(pos);
            return false;
        }
        return true;
    }
    template <class T>
    bool rd(T *out) {
        if (!need(sizeof(T))) return false;
        std::memcpy(out, p + pos, sizeof(T));
        pos += sizeof(T);
        return true;
    }
    bool str(std::string *out) {
        uint64_t len;
        if (!rd(&len)) return false;
        if (len > size - pos) {
            err = "GGUF string of " + std::to_string(len) + " bytes runs past the end of the file";
            return false;
        }
        out->assign(reinterpret_cast<const char *>(p + pos), (size_t)len);
        pos += (size_t)len;
        return true;
    }
    bool value_of(uint32_t type, GgufValue *v, int depth) {
        switch (type) {
        case 0: { uint8_t x; if (!rd(&x)) return false; v->kind = GgufValue::U8; v->u = x; return true; }
        case 1: { int8_t x; if (!rd(&x)) return false; v->kind = GgufValue::I8; v->i = x; return true; }
        case 2: { uint16_t x; if (!rd(&x)) return false; v->kind = GgufValue::U16; v->u = x; return true; }
        case 3: { int16_t x; if (!rd(&x)) return false; v->kind = GgufValue::I16; v->i = x; return true; }
        case 4: { uint32_t x; if (!rd(&x)) return false; v->kind = GgufValue::U32; v->u = x; return true; }
        case 5: { int32_t x; if (!rd(&x)) return false; v->kind = GgufValue::I32; v->i = x; return true; }
        case 6: { float x; if (!rd(&x)) return false; v->kind = GgufValue::F32; v->f = x; return true; }
        case 7: { uint8_t x; if (!rd(&x)) return false; v->kind = GgufValue::Bool; v->u = x != 0; return true; }
        case 8: v->kind = GgufValue::String; return str(&v->s);
        case 9: {
            uint32_t et;
            uint64_t len;
            if (!rd(&et) || !rd(&len)) return false;
            if (et > 12) {
                err = "unknown GGUF array element type code: " + std::to_string(et);
                return false;
            }
            if (depth > 4 || len > size - pos) {  // every element takes at least one byte
                err = "GGUF array of " + std::to_string(len) + " elements does not fit the file";
                return false;
            }
            v->kind = GgufValue::Array;
            v->arr.resize((size_t)len);
            for (auto &e : v->arr)
                if (!value_of(et, &e, depth + 1)) return false;
            return true;
        }
        case 10: { uint64_t x; if (!rd(&x)) return false; v->kind = GgufValue::U64; v->u = x; return true; }
        case 11: { int64_t x; if (!rd(&x)) return false; v->kind = GgufValue::I64; v->i = x; return true; }
        case 12: { double x; if (!rd(&x)) return false; v->kind = GgufValue::F64; v->f = x; return true; }
        default:
            err = "unknown GGUF metadata type code: " + std::to_string(type);
            return false;
        }
    }
};

}  // namespace

std::unique_ptr<GgufFile> GgufFile::load(const std::string &path, std::string *err) {
    std::unique_ptr<GgufFile> g(new GgufFile());
    if (!g->file_.open(path, err)) return nullptr;
    if (g->file_.size() < 16) {
        *err = "GGUF file too small";
        return nullptr;
    }
    Cursor c{g->file_.data(), g->file_.size()};
    uint32_t magic = 0;
    c.rd(&magic);
    if (magic != GGUF_MAGIC) {
        char buf[96];
        std::snprintf(buf, sizeof buf, "invalid GGUF magic: 0x%08X (expected 0x%08X)", magic, GGUF_MAGIC);
        *err = buf;
        return nullptr;
    }
    c.rd(&g->version_);
    if (g->version_ < 2 || g->version_ > 3) {
        *err = "unsupported GGUF version: " + std::to_string(g->version_) + " (expected 2 or 3)";
        return nullptr;
    }
    uint64_t n_tensors = 0, n_kv = 0;
    if (g->version_ >= 3) {  // v2 keeps the counts in 32 bits
        if (!c.rd(&n_tensors) || !c.rd(&n_kv)) { *err = c.err; return nullptr; }
    } else {
        uint32_t a, b;
        if (!c.rd(&a) || !c.rd(&b)) { *err = c.err; return nullptr; }
        n_tensors = a;
        n_kv = b;
    }
    if (n_tensors > c.size || n_kv > c.size) {
        *err = "GGUF header counts exceed the file size";
        return nullptr;
    }
    for (uint64_t i = 0; i < n_kv; i++) {
        std::string key;
        uint32_t type;
        GgufValue v;
        if (!c.str(&key) || !c.rd(&type) || !c.value_of(type, &v, 0)) { *err = c.err; return nullptr; }
        g->metadata_[key] = std::move(v);
    }
    size_t alignment = GGUF_DEFAULT_ALIGNMENT;
    if (const GgufValue *a = g->meta("general.alignment")) {
        uint64_t x;
        if (a->as_u64(&x) && x > 0 && (x & (x - 1)) == 0) alignment = (size_t)x;
    }
    g->tensors_.reserve((size_t)n_tensors);
    for (uint64_t i = 0; i < n_tensors; i++) {
        GgufTensorInfo t;
        uint32_t n_dims, code;
        if (!c.str(&t.name) || !c.rd(&n_dims)) { *err = c.err; return nullptr; }
        if (n_dims > 8) {
            *err = "tensor '" + t.name + "' has " + std::to_string(n_dims) + " dimensions";
            return nullptr;
        }
        t.shape.resize(n_dims);
        for (uint32_t d = 0; d < n_dims; d++)
            if (!c.rd(&t.shape[n_dims - 1 - d])) { *err = c.err; return nullptr; }  // innermost first in the file
        if (!c.rd(&code) || !c.rd(&t.offset)) { *err = c.err; return nullptr; }
        if (!ggml_type_known(code)) {
            *err = "unknown GGML type code " + std::to_string(code) + " for tensor '" + t.name + "'";
            return nullptr;
        }
        t.type = (GgmlType)code;
        if (t.num_elements() % ggml_block_size(t.type)) {
            *err = "tensor '" + t.name + "': element count is not a multiple of the " + ggml_type_name(t.type) + " block";
            return nullptr;
        }
        g->by_name_[t.name] = g->tensors_.size();
        g->tensors_.push_back(std::move(t));
    }
    g->data_offset_ = (c.pos + alignment - 1) & ~(alignment - 1);
    for (const auto &t : g->tensors_) {
        const size_t bytes = t.byte_size();
        if (g->data_offset_ > g->file_.size() || t.offset > g->file_.size() - g->data_offset_ ||
            bytes > g->file_.size() - g->data_offset_ - t.offset) {
            *err = "tensor '" + t.name + "' runs past the end of the file";
            return nullptr;
        }
    }
    return g;
}

const GgufTensorInfo *GgufFile::tensor_info(const std::string &name) const {
    auto it = by_name_.find(name);
    return it == by_name_.end() ? nullptr : &tensors_[it->second];
}
const uint8_t *GgufFile::tensor_data(const GgufTensorInfo &info) const {
    return file_.data() + data_offset_ + info.offset;
}
const GgufValue *GgufFile::meta(const std::string &key) const {
    auto it = metadata_.find(key);
    return it == metadata_.end() ? nullptr : &it->second;
}
bool GgufFile::architecture(std::string *out) const {
    const GgufValue *v = meta("general.architecture");
    return v && v->as_str(out);
}

bool GgufFile::transformer_config(TransformerConfig *cfg, std::string *err) const {
    std::string arch;
    if (!architecture(&arch)) {
        *err = "missing general.architecture metadata";
        return false;
    }
    auto get_u64 = [&](const std::string &key, uint64_t *out) {
        const GgufValue *v = meta(key);
        return v && v->as_u64(out);
    };
    auto need_u64 = [&](const std::string &key, uint64_t *out) {
        if (get_u64(key, out)) return true;
        *err = "missing or invalid metadata: " + key;
        return false;
    };
    auto get_f = [&](const std::string &key, double *out) {
        const GgufValue *v = meta(key);
        float f;
        if (!v || !v->as_f32(&f)) return false;
        *out = (double)f;
        return true;
    };
    uint64_t hidden, inter, heads, layers, x;
    if (!need_u64(arch + ".embedding_length", &hidden) || !need_u64(arch + ".feed_forward_length", &inter) ||
        !need_u64(arch + ".attention.head_count", &heads) || !need_u64(arch + ".block_count", &layers))
        return false;
    TransformerConfig c;
    c.hidden_size = (int)hidden;
    c.intermediate_size = (int)inter;
    c.num_attention_heads = (int)heads;
    c.num_hidden_layers = (int)layers;
    c.num_key_value_heads = get_u64(arch + ".attention.head_count_kv", &x) ? (int)x : 0;
    if (get_u64(arch + ".vocab_size", &x)) {
        c.vocab_size = (int)x;
    } else {  // fall back to the tokenizer's token count
        const GgufValue *tok = meta("tokenizer.ggml.tokens");
        if (!tok || tok->kind != GgufValue::Array) {
            *err = "cannot determine vocab_size";
            return false;
        }
        c.vocab_size = (int)tok->arr.size();
    }
    double f;
    c.rms_norm_eps = get_f(arch + ".attention.layer_norm_rms_epsilon", &f) ? f : 1e-6;
    c.rope_theta = get_f(arch + ".rope.freq_base", &f) ? f : 10000.0;
    c.max_position_embeddings = get_u64(arch + ".context_length", &x) ? (int)x : 2048;
    c.tie_word_embeddings = tensor_info("output.weight") == nullptr;
    c.head_dim_opt = get_u64(arch + ".attention.key_length", &x) ? (int)x : 0;
    c.attention_bias = tensor_info("blk.0.attn_q.bias") != nullptr;
    c.eos_token_id = get_u64("tokenizer.ggml.eos_token_id", &x) ? (int)x : -1;
    c.bos_token_id = get_u64("tokenizer.ggml.bos_token_id", &x) ? (int)x : -1;
    *cfg = c;
    return true;
}

// ── tensors -> host arrays in the layouts set_weight takes ───────────────────

namespace {

// any supported GGML type -> f32 (reference load_f32_buffer, src/gguf.rs:726-775; plus Q4_0)
}  // namespace

bool ggml_to_f32(GgmlType type, const uint8_t *src, size_t n, std::vector<float> *out, std::string *err) {
    out->resize(n);
    float *dst = out->data();
    switch (type) {
    case GgmlType::F32: std::memcpy(dst, src, n * 4); return true;
    case GgmlType::F16:
        for (size_t i = 0; i < n; i++) dst[i] = f16_bits_to_f32_host(rd16(src + 2 * i));
        return true;
    case GgmlType::BF16:
        for (size_t i = 0; i < n; i++) dst[i] = bf16_bits_to_f32_host(rd16(src + 2 * i));
        return true;
    case GgmlType::Q8_0: dequant_q8_0_host(src, dst, n); return true;
    case GgmlType::Q4_0: dequant_q4_0_host(src, dst, n); return true;
    case GgmlType::Q4K:
    case GgmlType::Q6K:
        if (n % 256 != 0) {
            *err = std::string(ggml_type_name(type)) + " tensor whose size is not a multiple of 256";
            return false;
        }
        if (type == GgmlType::Q4K)
            dequant_q4_k_host(src, dst, n);
        else
            dequant_q6_k_host(src, dst, n);
        return true;
    default:
        *err = std::string("unsupported type ") + ggml_type_name(type) + " for an f32 tensor";
        return false;
    }
}

namespace {

// F32 / F16 / BF16 -> bf16 bits (F32 by truncation, as the reference's bf16 plan does)
bool ggml_to_bf16(GgmlType type, const uint8_t *src, size_t n, std::vector<uint16_t> *out, std::string *err) {
    out->resize(n);
    uint16_t *dst = out->data();
    switch (type) {
    case GgmlType::BF16: std::memcpy(dst, src, n * 2); return true;
    case GgmlType::F32:
        for (size_t i = 0; i < n; i++) {
            float f;
            std::memcpy(&f, src + 4 * i, 4);
            dst[i] = f32_to_bf16_trunc_host(f);
        }
        return true;
    case GgmlType::F16:
        for (size_t i = 0; i < n; i++) dst[i] = f32_to_bf16_trunc_host(f16_bits_to_f32_host(rd16(src + 2 * i)));
        return true;
    default:
        *err = std::string("unsupported type ") + ggml_type_name(type) + " for a bf16 projection";
        return false;
    }
}

// "model.layers.3.self_attn.q_proj.weight" -> "blk.3.attn_q.weight" (names of src/gguf.rs:618-680)
std::string gguf_name_of(const std::string &hf) {
    if (hf == "model.embed_tokens.weight") return "token_embd.weight";
    if (hf == "model.norm.weight") return "output_norm.weight";
    if (hf == "lm_head.weight") return "output.weight";
    const std::string pre = "model.layers.";
    if (hf.compare(0, pre.size(), pre) != 0) return "";
    const size_t dot = hf.find('.', pre.size());
    if (dot == std::string::npos) return "";
    const std::string layer = hf.substr(pre.size(), dot - pre.size()), rest = hf.substr(dot + 1);
    static const std::pair<const char *, const char *> table[] = {
        {"input_layernorm.weight", "attn_norm.weight"},
        {"self_attn.q_proj.weight", "attn_q.weight"}, {"self_attn.q_proj.bias", "attn_q.bias"},
        {"self_attn.k_proj.weight", "attn_k.weight"}, {"self_attn.k_proj.bias", "attn_k.bias"},
        {"self_attn.v_proj.weight", "attn_v.weight"}, {"self_attn.v_proj.bias", "attn_v.bias"},
        {"self_attn.q_norm.weight", "attn_q_norm.weight"}, {"self_attn.k_norm.weight", "attn_k_norm.weight"},
        {"self_attn.o_proj.weight", "attn_output.weight"},
        {"post_attention_layernorm.weight", "ffn_norm.weight"},
        {"mlp.gate_proj.weight", "ffn_gate.weight"}, {"mlp.up_proj.weight", "ffn_up.weight"},
        {"mlp.down_proj.weight", "ffn_down.weight"},
    };
    for (const auto &e : table)
        if (rest == e.first) return "blk." + layer + "." + e.second;
    return "";
}

bool is_projection(const std::string &hf_name) {
    return hf_name.size() > 12 && hf_name.compare(hf_name.size() - 12, 12, "_proj.weight") == 0;
}

int fail(hm_ctx *ctx, const std::string &msg) { return hm_set_error(ctx, HM_ERR_INVALID, "%s", msg.c_str()); }

int pick_seq_len(const TransformerConfig &cfg, int max_seq_len) {
    if (max_seq_len > 0) return max_seq_len;
    return cfg.max_position_embeddings < 4096 ? cfg.max_position_embeddings : 4096;
}

}  // namespace

std::unique_ptr<HfModel> load_gguf_model(hm_ctx *ctx, const std::string &path, int max_seq_len) {
    std::string err;
    std::unique_ptr<GgufFile> g = GgufFile::load(path, &err);
    if (!g) {
        fail(ctx, path + ": " + err);
        return nullptr;
    }
    TransformerConfig cfg;
    if (!g->transformer_config(&cfg, &err)) {
        fail(ctx, path + ": " + err);
        return nullptr;
    }
    const bool has_qk_norm = g->tensor_info("blk.0.attn_q_norm.weight") != nullptr;
    // Every projection carries its own type (reference Buffer dtype from GgmlType::to_dtype,
    // src/gguf.rs:593-613); a file is either block-quantised throughout (types may differ per matrix,
    // as in Q4_K_M files) or float throughout.
    static const char *const proj_names[7] = {"attn_q", "attn_k", "attn_v", "attn_output", "ffn_gate", "ffn_up", "ffn_down"};
    std::vector<DType> proj_dtypes;
    int n_float = 0;
    for (int l = 0; l < cfg.num_hidden_layers; l++)
        for (int j = 0; j < 7; j++) {
            const std::string name = "blk." + std::to_string(l) + "." + proj_names[j] + ".weight";
            const GgufTensorInfo *t = g->tensor_info(name);
            if (!t) {
                fail(ctx, path + ": missing GGUF tensor: " + name);
                return nullptr;
            }
            switch (t->type) {
            case GgmlType::Q8_0: proj_dtypes.push_back(DType::Q8_0); break;
            case GgmlType::Q4_0: proj_dtypes.push_back(DType::Q4_0); break;
            case GgmlType::Q4K: proj_dtypes.push_back(DType::Q4_K); break;
            case GgmlType::Q6K: proj_dtypes.push_back(DType::Q6_K); break;
            case GgmlType::F32: case GgmlType::F16: case GgmlType::BF16:
                proj_dtypes.push_back(DType::BF16);
                n_float++;
                break;
            default:
                fail(ctx, path + ": tensor " + name + " is " + ggml_type_name(t->type) +
                              "; this build runs Q8_0, Q4_0, Q4_K, Q6_K and F32/F16/BF16 projections");
                return nullptr;
            }
        }
    if (proj_dtypes.empty()) {
        fail(ctx, path + ": the model has no layers");
        return nullptr;
    }
    if (n_float != 0 && n_float != (int)proj_dtypes.size()) {
        fail(ctx, path + ": some projections are block-quantised and some are float (mixing the two is not supported)");
        return nullptr;
    }
    const bool quant = n_float == 0;
    std::unique_ptr<HfModel> m = quant ? HfModel::create(ctx, cfg, proj_dtypes[0], has_qk_norm, &proj_dtypes)
                                       : HfModel::create(ctx, cfg, DType::BF16, has_qk_norm);
    if (!m) return nullptr;

    std::vector<float> f32;
    std::vector<uint16_t> b16;
    const auto &slots = m->weight_slot_infos();
    for (size_t i = 0; i < slots.size(); i++) {
        const WeightSlotInfo &slot = slots[i];
        std::string name = gguf_name_of(slot.name);
        if (slot.name == "lm_head.weight" && cfg.tie_word_embeddings) name = "token_embd.weight";
        const GgufTensorInfo *t = name.empty() ? nullptr : g->tensor_info(name);
        if (!t) {
            fail(ctx, path + ": missing GGUF tensor: " + (name.empty() ? slot.name : name));
            return nullptr;
        }
        const uint8_t *src = g->tensor_data(*t);
        const size_t n = (size_t)t->num_elements();
        int rc;
        if (is_projection(slot.name)) {
            // GGUF keeps a projection as [out, in] rows: dim0/dim1 of a quantised slot, dim1/dim0 of a bf16 one
            const uint64_t rows = quant ? slot.dim0 : slot.dim1, cols = quant ? slot.dim1 : slot.dim0;
            if (t->shape.size() != 2 || t->shape[0] != rows || t->shape[1] != cols) {
                fail(ctx, path + ": tensor " + name + " does not have the shape [" + std::to_string(rows) + ", " +
                              std::to_string(cols) + "] the config implies");
                return nullptr;
            }
            if (quant) {
                rc = m->set_weight((int)i, src, t->byte_size());
            } else {
                if (!ggml_to_bf16(t->type, src, n, &b16, &err)) {
                    fail(ctx, path + ": tensor " + name + ": " + err);
                    return nullptr;
                }
                rc = m->set_weight_nk((int)i, b16.data(), n * 2);
            }
        } else if (slot.name == "lm_head.weight") {
            if (t->shape.size() != 2 || (int64_t)t->shape[0] != cfg.vocab_size || (int64_t)t->shape[1] != cfg.hidden_size) {
                fail(ctx, path + ": tensor " + name + " is not [vocab, hidden]");
                return nullptr;
            }
            const bool k_head = t->type == GgmlType::Q4K || t->type == GgmlType::Q6K;
            const bool b32_head = t->type == GgmlType::Q8_0 || t->type == GgmlType::Q4_0;
            if (quant && (k_head || b32_head) && cfg.hidden_size % (k_head ? 256 : 32) == 0 && cfg.hidden_size <= 4096) {
                // the f32 head of the quantised plan (src/gguf.rs:696-700), taken from the blocks as they are
                const DType hd = t->type == GgmlType::Q6K ? DType::Q6_K : t->type == GgmlType::Q4K ? DType::Q4_K
                                 : t->type == GgmlType::Q8_0 ? DType::Q8_0 : DType::Q4_0;
                rc = m->set_lm_head_blocks(hd, src, t->byte_size());
            } else if (quant) {  // the quantised plan keeps an f32 head (src/gguf.rs:696-700)
                if (!ggml_to_f32(t->type, src, n, &f32, &err)) {
                    fail(ctx, path + ": tensor " + name + ": " + err);
                    return nullptr;
                }
                rc = m->set_weight_nk((int)i, f32.data(), n * 4);
            } else {
                if (t->type == GgmlType::Q8_0 || t->type == GgmlType::Q4_0 || t->type == GgmlType::Q4K ||
                    t->type == GgmlType::Q6K) {
                    if (!ggml_to_f32(t->type, src, n, &f32, &err)) {
                        fail(ctx, path + ": tensor " + name + ": " + err);
                        return nullptr;
                    }
                    b16.resize(n);
                    for (size_t k = 0; k < n; k++) b16[k] = f32_to_bf16_trunc_host(f32[k]);
                } else if (!ggml_to_bf16(t->type, src, n, &b16, &err)) {
                    fail(ctx, path + ": tensor " + name + ": " + err);
                    return nullptr;
                }
                rc = m->set_weight_nk((int)i, b16.data(), n * 2);
            }
        } else {  // embedding, norms, biases: f32
            if (n * 4 != slot.bytes) {
                fail(ctx, path + ": tensor " + name + " has " + std::to_string(n) + " elements, the config implies " +
                              std::to_string(slot.bytes / 4));
                return nullptr;
            }
            if (!ggml_to_f32(t->type, src, n, &f32, &err)) {
                fail(ctx, path + ": tensor " + name + ": " + err);
                return nullptr;
            }
            rc = m->set_weight((int)i, f32.data(), n * 4);
        }
        if (rc != HM_OK) return nullptr;
    }
    if (m->finalize(pick_seq_len(cfg, max_seq_len)) != HM_OK) return nullptr;
    return m;
}

// ── files ───────────────────────────────────────────────────────────────────

namespace {

bool read_text_file(const std::string &path, std::string *out, std::string *err) {
    MappedFile f;
    if (!f.open(path, err)) return false;
    out->assign(reinterpret_cast<const char *>(f.data()), f.size());
    return true;
}

bool file_exists(const std::string &path) {
    struct stat st;
    return stat(path.c_str(), &st) == 0 && S_ISREG(st.st_mode);
}

}  // namespace

bool parse_json_string_to_int_map(const char *text, size_t len, std::vector<std::pair<std::string, int64_t>> *out,
                                  std::string *err) {
    Json j;
    if (!parse_json(text, len, &j, err)) return false;
    if (j.kind != Json::Obj) {
        *err = "JSON: expected an object of string -> integer";
        return false;
    }
    out->clear();
    out->reserve(j.obj.size());
    for (auto &kv : j.obj) {
        if (kv.second.kind != Json::Num || kv.second.num != std::floor(kv.second.num)) {
            *err = "JSON: value of \"" + kv.first + "\" is not an integer";
            return false;
        }
        out->emplace_back(std::move(kv.first), (int64_t)kv.second.num);
    }
    return true;
}


bool transformer_config_from_json(const std::string &text, TransformerConfig *cfg, std::string *err) {
    Json j;
    if (!parse_json(text.data(), text.size(), &j, err)) return false;
    if (j.kind != Json::Obj) {
        *err = "config.json: not an object";
        return false;
    }
    auto need_int = [&](const char *key, int *out) {
        const Json *v = j.get(key);
        if (!v || v->kind != Json::Num || v->num < 0 || v->num != std::floor(v->num)) {
            *err = std::string("config.json: missing field `") + key + "`";  // serde: "missing field `x`"
            return false;
        }
        *out = (int)v->num;
        return true;
    };
    TransformerConfig c;
    if (!need_int("hidden_size", &c.hidden_size) || !need_int("intermediate_size", &c.intermediate_size) ||
        !need_int("num_attention_heads", &c.num_attention_heads) || !need_int("num_hidden_layers", &c.num_hidden_layers) ||
        !need_int("vocab_size", &c.vocab_size))
        return false;
    auto opt_num = [&](const char *key, double *out) {
        const Json *v = j.get(key);
        if (!v || v->kind != Json::Num) return false;
        *out = v->num;
        return true;
    };
    double x;
    c.num_key_value_heads = opt_num("num_key_value_heads", &x) ? (int)x : 0;
    c.rms_norm_eps = opt_num("rms_norm_eps", &x) ? x : 1e-6;
    c.rope_theta = opt_num("rope_theta", &x) ? x : 10000.0;
    c.max_position_embeddings = opt_num("max_position_embeddings", &x) ? (int)x : 2048;
    c.head_dim_opt = opt_num("head_dim", &x) ? (int)x : 0;
    const Json *tie = j.get("tie_word_embeddings");
    c.tie_word_embeddings = tie && tie->kind == Json::Bool && tie->b;
    c.eos_token_id = opt_num("eos_token_id", &x) && x >= 0 ? (int)x : -1;
    c.bos_token_id = opt_num("bos_token_id", &x) && x >= 0 ? (int)x : -1;
    *cfg = c;
    return true;
}

// ── safetensors ──────────────────────────────────────────────────────────────

std::unique_ptr<SafeTensorsFile> SafeTensorsFile::load(const std::string &path, std::string *err) {
    std::unique_ptr<SafeTensorsFile> s(new SafeTensorsFile());
    if (!s->file_.open(path, err)) return nullptr;
    const size_t size = s->file_.size();
    if (size < 8) {
        *err = "safetensors file too small (< 8 bytes)";
        return nullptr;
    }
    uint64_t header_len;
    std::memcpy(&header_len, s->file_.data(), 8);
    if (header_len > size - 8) {
        *err = "safetensors header length " + std::to_string(header_len) + " exceeds file size " + std::to_string(size);
        return nullptr;
    }
    Json j;
    if (!parse_json(reinterpret_cast<const char *>(s->file_.data() + 8), (size_t)header_len, &j, err)) return nullptr;
    if (j.kind != Json::Obj) {
        *err = "safetensors header is not a JSON object";
        return nullptr;
    }
    s->data_base_ = 8 + (size_t)header_len;
    const size_t data_size = size - s->data_base_;
    for (const auto &kv : j.obj) {
        if (kv.first == "__metadata__") continue;
        const Json *dt = kv.second.get("dtype"), *sh = kv.second.get("shape"), *off = kv.second.get("data_offsets");
        if (!dt || dt->kind != Json::Str || !sh || sh->kind != Json::Arr || !off || off->kind != Json::Arr ||
            off->arr.size() != 2 || off->arr[0].kind != Json::Num || off->arr[1].kind != Json::Num) {
            *err = "safetensors: malformed entry for tensor '" + kv.first + "'";
            return nullptr;
        }
        SafeTensorInfo t;
        t.name = kv.first;
        t.dtype = dt->str;
        for (const Json &d : sh->arr) {
            if (d.kind != Json::Num || d.num < 0) {
                *err = "safetensors: bad shape for tensor '" + kv.first + "'";
                return nullptr;
            }
            t.shape.push_back((uint64_t)d.num);
        }
        if (t.shape.size() > 8) {  // as the GGUF reader: the C boundary reports at most eight dimensions
            *err = "safetensors: tensor '" + kv.first + "' has " + std::to_string(t.shape.size()) + " dimensions";
            return nullptr;
        }
        t.begin = (size_t)off->arr[0].num;
        t.end = (size_t)off->arr[1].num;
        if (t.begin > t.end || t.end > data_size) {
            *err = "safetensors: tensor '" + kv.first + "' runs past the end of the file";
            return nullptr;
        }
        s->by_name_[t.name] = s->tensors_.size();
        s->tensors_.push_back(std::move(t));
    }
    return s;
}

const SafeTensorInfo *SafeTensorsFile::find(const std::string &name) const {
    auto it = by_name_.find(name);
    return it == by_name_.end() ? nullptr : &tensors_[it->second];
}

namespace {

size_t st_elem_size(const std::string &dtype) {
    if (dtype == "F32" || dtype == "I32") return 4;
    if (dtype == "BF16" || dtype == "F16") return 2;
    if (dtype == "F64" || dtype == "I64") return 8;
    return 0;
}

bool st_to_f32(const SafeTensorInfo &t, const uint8_t *src, std::vector<float> *out, std::string *err) {
    const size_t es = st_elem_size(t.dtype);
    const size_t n = es ? (t.end - t.begin) / es : 0;
    out->resize(n);
    if (t.dtype == "F32") {
        std::memcpy(out->data(), src, n * 4);
    } else if (t.dtype == "BF16") {
        for (size_t i = 0; i < n; i++) (*out)[i] = bf16_bits_to_f32_host(rd16(src + 2 * i));
    } else if (t.dtype == "F16") {
        for (size_t i = 0; i < n; i++) (*out)[i] = f16_bits_to_f32_host(rd16(src + 2 * i));
    } else if (t.dtype == "F64") {
        for (size_t i = 0; i < n; i++) {
            double d;
            std::memcpy(&d, src + 8 * i, 8);
            (*out)[i] = (float)d;
        }
    } else {
        *err = "unsupported safetensors dtype: " + t.dtype;  // reference src/hf/safetensors.rs:88-90
        return false;
    }
    return true;
}

bool st_to_bf16(const SafeTensorInfo &t, const uint8_t *src, std::vector<uint16_t> *out, std::string *err) {
    if (t.dtype == "BF16") {
        const size_t n = (t.end - t.begin) / 2;
        out->resize(n);
        std::memcpy(out->data(), src, n * 2);
        return true;
    }
    std::vector<float> f;
    if (!st_to_f32(t, src, &f, err)) return false;
    out->resize(f.size());
    for (size_t i = 0; i < f.size(); i++) (*out)[i] = f32_to_bf16_trunc_host(f[i]);
    return true;
}

}  // namespace

std::unique_ptr<HfModel> load_hf_model_dir(hm_ctx *ctx, const std::string &dir, int max_seq_len) {
    std::string err, text;
    if (!read_text_file(dir + "/config.json", &text, &err)) {
        fail(ctx, err);
        return nullptr;
    }
    TransformerConfig cfg;
    if (!transformer_config_from_json(text, &cfg, &err)) {
        fail(ctx, dir + "/config.json: " + err);
        return nullptr;
    }
    // one file, or the shards a model.safetensors.index.json names (reference src/hf/model.rs:86-123)
    std::vector<std::unique_ptr<SafeTensorsFile>> files;
    if (file_exists(dir + "/model.safetensors")) {
        auto f = SafeTensorsFile::load(dir + "/model.safetensors", &err);
        if (!f) {
            fail(ctx, dir + "/model.safetensors: " + err);
            return nullptr;
        }
        files.push_back(std::move(f));
    } else if (file_exists(dir + "/model.safetensors.index.json")) {
        Json idx;
        if (!read_text_file(dir + "/model.safetensors.index.json", &text, &err) ||
            !parse_json(text.data(), text.size(), &idx, &err)) {
            fail(ctx, dir + "/model.safetensors.index.json: " + err);
            return nullptr;
        }
        const Json *map = idx.get("weight_map");
        if (!map || map->kind != Json::Obj) {
            fail(ctx, "model.safetensors.index.json missing weight_map");
            return nullptr;
        }
        std::set<std::string> shards;
        for (const auto &kv : map->obj)
            if (kv.second.kind == Json::Str) shards.insert(kv.second.str);
        for (const std::string &name : shards) {
            if (name.find('/') != std::string::npos || name.find("..") != std::string::npos) {
                fail(ctx, "model.safetensors.index.json names a shard outside the model directory: " + name);
                return nullptr;
            }
            auto f = SafeTensorsFile::load(dir + "/" + name, &err);
            if (!f) {
                fail(ctx, dir + "/" + name + ": " + err);
                return nullptr;
            }
            files.push_back(std::move(f));
        }
    } else {
        fail(ctx, "no model.safetensors or index found in " + dir);
        return nullptr;
    }
    auto find = [&](const std::string &name, const SafeTensorsFile **owner) -> const SafeTensorInfo * {
        for (const auto &f : files)
            if (const SafeTensorInfo *t = f->find(name)) {
                *owner = f.get();
                return t;
            }
        return nullptr;
    };
    const SafeTensorsFile *owner = nullptr;
    cfg.attention_bias = find("model.layers.0.self_attn.q_proj.bias", &owner) != nullptr;
    const bool has_qk_norm = find("model.layers.0.self_attn.q_norm.weight", &owner) != nullptr;
    const bool own_head = find("lm_head.weight", &owner) != nullptr;

    std::unique_ptr<HfModel> m = HfModel::create(ctx, cfg, DType::BF16, has_qk_norm);
    if (!m) return nullptr;
    std::vector<float> f32;
    std::vector<uint16_t> b16;
    const auto &slots = m->weight_slot_infos();
    for (size_t i = 0; i < slots.size(); i++) {
        const WeightSlotInfo &slot = slots[i];
        // no lm_head tensor: the head is the embedding (src/hf/weights.rs:101-113)
        const std::string name = (slot.name == "lm_head.weight" && !own_head) ? "model.embed_tokens.weight" : slot.name;
        const SafeTensorInfo *t = find(name, &owner);
        if (!t) {
            fail(ctx, "missing weight: " + name);
            return nullptr;
        }
        const uint8_t *src = owner->data(*t);
        const size_t es = st_elem_size(t->dtype);
        if (!es) {
            fail(ctx, "unsupported safetensors dtype: " + t->dtype);
            return nullptr;
        }
        const size_t n = (t->end - t->begin) / es;
        uint64_t want = 1;
        for (uint64_t d : t->shape) want *= d;
        if (want != n) {
            fail(ctx, "tensor " + name + ": data size does not match its shape");
            return nullptr;
        }
        int rc;
        if (slot.dtype == DType::BF16) {  // projections and LM head: HF keeps them [out, in] = [N][K]
            if (t->shape.size() != 2 || (int64_t)t->shape[0] != slot.dim1 || (int64_t)t->shape[1] != slot.dim0) {
                fail(ctx, "tensor " + name + " does not have the shape [" + std::to_string(slot.dim1) + ", " +
                              std::to_string(slot.dim0) + "] the config implies");
                return nullptr;
            }
            if (!st_to_bf16(*t, src, &b16, &err)) {
                fail(ctx, "tensor " + name + ": " + err);
                return nullptr;
            }
            rc = m->set_weight_nk((int)i, b16.data(), n * 2);
        } else {
            if (n * 4 != slot.bytes) {
                fail(ctx, "tensor " + name + " has " + std::to_string(n) + " elements, the config implies " +
                              std::to_string(slot.bytes / 4));
                return nullptr;
            }
            if (!st_to_f32(*t, src, &f32, &err)) {
                fail(ctx, "tensor " + name + ": " + err);
                return nullptr;
            }
            rc = m->set_weight((int)i, f32.data(), n * 4);
        }
        if (rc != HM_OK) return nullptr;
    }
    if (m->finalize(pick_seq_len(cfg, max_seq_len)) != HM_OK) return nullptr;
    return m;
}

}  // namespace homura
