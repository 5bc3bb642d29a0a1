// Byte-level BPE tokenizer over vocab.json + merges.txt: the reference's own Tokenizer
// (src/tokenizer.rs:6-158). Host code only.
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
    // reference encode (src/tokenizer.rs:119-144): pieces of the pre-tokeniser pattern, bytes mapped to
    // printable code points, merges by rank; pieces missing from the vocabulary are dropped
    std::vector<uint32_t> encode(const char *text, size_t len) const;
    // reference decode (src/tokenizer.rs:147-159): unknown ids and unmapped characters are dropped,
    // invalid UTF-8 becomes U+FFFD
    std::string decode(const uint32_t *ids, size_t n) const;
    size_t vocab_size() const { return encoder_.size(); }

    // [begin, end) byte ranges of the pieces the pre-tokeniser pattern cuts text into (exposed for tests)
    static std::vector<std::pair<size_t, size_t>> pre_tokenize(const char *text, size_t len);

private:
    std::vector<std::string> bpe(const std::string &mapped) const;
    std::unordered_map<std::string, uint32_t> encoder_;
    std::unordered_map<uint32_t, std::string> decoder_;
    std::unordered_map<std::string, uint32_t> ranks_;  // "left right" -> rank
    std::string byte_utf8_[256];                       // byte -> UTF-8 of its printable stand-in
    std::unordered_map<uint32_t, uint8_t> cp_to_byte_;
};

}  // namespace homura
