// BPE tokenizer. Sources: vocab.json + merges.txt, the reference's own byte-level Tokenizer
// (src/tokenizer.rs:6-158); a tokenizer.json of the byte-level BPE family (Qwen2/3, Llama-3) or of the
// SentencePiece-style BPE family (Llama-2, TinyLlama, Mistral: "\u2581" for spaces, byte fallback), which the
// reference hands to the `tokenizers` crate (HfTokenizer, src/hf/tokenizer.rs:4-47). Host code only.
#pragma once

#include <cstdint>
#include <memory>
#include <string>
#include <unordered_map>
#include <vector>

namespace homura {

class BpeTokenizer {
public:
    // reference Tokenizer::from_files (src/tokenizer.rs:44-82)
    static std::unique_ptr<BpeTokenizer> from_files(const std::string &vocab_path, const std::string &merges_path,
                                                    std::string *err);
    // HfTokenizer::from_file (src/hf/tokenizer.rs:10-14) for the files this class can honour: model BPE
    // without unknown-token or byte fallback, ByteLevel pre-tokeniser and decoder behind a Split on the
    // Qwen2 or Llama-3 pattern, added tokens without strip or single-word flags, post-processor ByteLevel
    // or TemplateProcessing. Or: model BPE with unk_token, fuse_unk and byte_fallback, normaliser
    // Sequence[Prepend("\u2581"), Replace(" " -> "\u2581")], no pre-tokeniser, decoder Sequence[Replace("\u2581" -> " "),
    // ByteFallback, Fuse, Strip(" ", 1, 0)] (the Llama-2 family). Anything else is refused with a message. An NFC
    // normaliser is recorded (wants_nfc) and left to the caller: this class does not normalise.
    static std::unique_ptr<BpeTokenizer> from_tokenizer_json(const std::string &path, std::string *err);
    // reference encode (src/tokenizer.rs:119-144): pieces of the pre-tokeniser pattern, bytes mapped to
    // printable code points, merges by rank; pieces missing from the vocabulary are dropped. Added tokens
    // (tokenizer.json) are cut out of the text first, leftmost and longest, and stand for themselves;
    // add_special_tokens puts the post-processor's template around the ids (HfTokenizer::encode_with_special,
    // src/hf/tokenizer.rs:41-47).
    std::vector<uint32_t> encode(const char *text, size_t len, bool add_special_tokens = false) const;
    // reference decode (src/tokenizer.rs:147-159): unknown ids and unmapped characters are dropped,
    // invalid UTF-8 becomes U+FFFD. tokenizer.json: a token with a character outside the byte alphabet
    // contributes its own UTF-8 bytes; skip_special drops added tokens marked special
    // (HfTokenizer::decode / decode_raw, src/hf/tokenizer.rs:25-38).
    std::string decode(const uint32_t *ids, size_t n, bool skip_special = false) const;
    size_t vocab_size() const { return decoder_.size(); }
    // id of a vocabulary entry or added token, -1 when absent
    int64_t token_to_id(const std::string &token) const;
    bool wants_nfc() const { return wants_nfc_; }

    // [begin, end) byte ranges of the pieces the pre-tokeniser pattern cuts text into (exposed for tests);
    // max_digits = longest run of numbers in one piece (3: the reference's pattern and Llama-3; 1: Qwen2)
    static std::vector<std::pair<size_t, size_t>> pre_tokenize(const char *text, size_t len, int max_digits = 3);

private:
    struct Added {
        std::string content;
        uint32_t id;
        bool special;
    };
    void init_byte_alphabet();
    void encode_plain(const char *text, size_t len, std::vector<uint32_t> *ids) const;
    // the SentencePiece-style family: the whole stretch is one word of characters (bytes where a character is not
    // in the vocabulary), merged by rank
    void encode_plain_spm(const char *text, size_t len, std::vector<uint32_t> *ids) const;
    std::string decode_spm(const uint32_t *ids, size_t n, bool skip_special) const;
    bool spm_ = false;            // SentencePiece-style family
    int64_t unk_id_ = -1;
    int64_t byte_ids_[256];       // ids of "<0x00>" .. "<0xFF>", -1 when absent
    std::vector<Added> added_;                         // longest content first
    std::unordered_map<uint32_t, size_t> added_by_id_;
    std::vector<uint32_t> prefix_ids_, suffix_ids_;    // post-processor template around a single sequence
    int max_digits_ = 3;
    bool ignore_merges_ = false;  // a piece that is a vocabulary entry is taken whole (Llama-3)
    bool hf_decode_ = false;
    bool wants_nfc_ = false;
    std::vector<std::string> bpe(const std::string &mapped) const;
    std::unordered_map<std::string, uint32_t> encoder_;
    std::unordered_map<uint32_t, std::string> decoder_;
    std::unordered_map<std::string, uint32_t> ranks_;  // "left right" -> rank
    std::string byte_utf8_[256];                       // byte -> UTF-8 of its printable stand-in
    std::unordered_map<uint32_t, uint8_t> cp_to_byte_;
};

}  // namespace homura
