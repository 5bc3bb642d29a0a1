// Byte-level BPE tokenizer (reference src/tokenizer.rs). The reference cuts the text with the regex
//   (?i:'s|'t|'re|'ve|'m|'ll|'d) | [^\r\n\p{L}\p{N}]?\p{L}+ | \p{N}{1,3} | ' '?[^\s\p{L}\p{N}]+[\r\n]* |
//   \s*[\r\n]+ | \s+(?!\S) | \s+
// (src/tokenizer.rs:71-74, first alternative that matches wins, each greedy with backtracking); here the
// seven alternatives are a hand-written scanner over code points, with the letter and number classes
// from generated range tables.
#include "tokenizer.h"

#include <cctype>
#include <cstdio>
#include <queue>

#include <algorithm>
#include <cstdio>
#include <cstring>
#include <fstream>
#include <sstream>

#include "../../../include/homura_amd.h"
#include "json.h"
#include "unicode_tables.h"

namespace homura {

namespace {

template <size_t N>
bool in_ranges(const uint32_t (&table)[N][2], uint32_t cp) {
    size_t lo = 0, hi = N;
    while (lo < hi) {
        const size_t mid = (lo + hi) / 2;
        if (cp < table[mid][0])
            hi = mid;
        else if (cp > table[mid][1])
            lo = mid + 1;
        else
            return true;
    }
    return false;
}

bool is_letter(uint32_t cp) { return in_ranges(UNICODE_LETTER_RANGES, cp); }
bool is_number(uint32_t cp) { return in_ranges(UNICODE_NUMBER_RANGES, cp); }
// the White_Space property, which is what \s means in the reference's regex engine
bool is_space(uint32_t cp) {
    return (cp >= 9 && cp <= 13) || cp == 0x20 || cp == 0x85 || cp == 0xA0 || cp == 0x1680 || (cp >= 0x2000 && cp <= 0x200A) ||
           cp == 0x2028 || cp == 0x2029 || cp == 0x202F || cp == 0x205F || cp == 0x3000;
}
bool is_newline(uint32_t cp) { return cp == '\r' || cp == '\n'; }

void append_utf8(std::string *out, uint32_t cp) {
    if (cp < 0x80) {
        out->push_back((char)cp);
    } else if (cp < 0x800) {
        out->push_back((char)(0xC0 | (cp >> 6)));
        out->push_back((char)(0x80 | (cp & 0x3F)));
    } else if (cp < 0x10000) {
        out->push_back((char)(0xE0 | (cp >> 12)));
        out->push_back((char)(0x80 | ((cp >> 6) & 0x3F)));
        out->push_back((char)(0x80 | (cp & 0x3F)));
    } else {
        out->push_back((char)(0xF0 | (cp >> 18)));
        out->push_back((char)(0x80 | ((cp >> 12) & 0x3F)));
        out->push_back((char)(0x80 | ((cp >> 6) & 0x3F)));
        out->push_back((char)(0x80 | (cp & 0x3F)));
    }
}

// Length of the well-formed UTF-8 sequence at s (0 if there is none) and its code point. `bad` receives
// how many bytes form the longest prefix of a well-formed sequence (at least 1), the unit that
// lossy decoding replaces by one U+FFFD.
size_t utf8_at(const unsigned char *s, size_t n, uint32_t *cp, size_t *bad) {
    const unsigned char b0 = s[0];
    *bad = 1;
    if (b0 < 0x80) {
        *cp = b0;
        return 1;
    }
    size_t need;
    unsigned char lo = 0x80, hi = 0xBF;
    uint32_t v;
    if (b0 >= 0xC2 && b0 <= 0xDF) {
        need = 1;
        v = b0 & 0x1F;
    } else if (b0 >= 0xE0 && b0 <= 0xEF) {
        need = 2;
        v = b0 & 0x0F;
        if (b0 == 0xE0) lo = 0xA0;
        if (b0 == 0xED) hi = 0x9F;
    } else if (b0 >= 0xF0 && b0 <= 0xF4) {
        need = 3;
        v = b0 & 0x07;
        if (b0 == 0xF0) lo = 0x90;
        if (b0 == 0xF4) hi = 0x8F;
    } else {
        return 0;
    }
    for (size_t k = 1; k <= need; k++) {
        if (k >= n || s[k] < lo || s[k] > hi) {
            *bad = k;
            return 0;
        }
        v = (v << 6) | (s[k] & 0x3F);
        lo = 0x80;
        hi = 0xBF;
    }
    *cp = v;
    return need + 1;
}

struct CodePoints {
    std::vector<uint32_t> cp;
    std::vector<size_t> at;  // byte offset of each code point, plus the total length at the end
};

// A byte that is not part of well-formed UTF-8 counts as one character of no class (U+FFFD); the
// piece still carries the original byte.
CodePoints decode_code_points(const char *text, size_t len) {
    CodePoints r;
    const unsigned char *s = reinterpret_cast<const unsigned char *>(text);
    size_t i = 0;
    while (i < len) {
        uint32_t cp;
        size_t bad;
        const size_t n = utf8_at(s + i, len - i, &cp, &bad);
        r.at.push_back(i);
        r.cp.push_back(n ? cp : 0xFFFD);
        i += n ? n : 1;
    }
    r.at.push_back(len);
    return r;
}

// End (exclusive, in code points) of the piece that starts at i.
size_t match_piece(const std::vector<uint32_t> &c, size_t i, int max_digits) {
    const size_t n = c.size();
    const uint32_t c0 = c[i];
    auto lower = [](uint32_t x) { return x >= 'A' && x <= 'Z' ? x + 32 : x; };
    // 1. contractions, case-insensitive (U+017F, the long s, folds to s)
    if (c0 == '\'' && i + 1 < n) {
        const uint32_t a = c[i + 1] == 0x17F ? 's' : lower(c[i + 1]);
        const uint32_t b = i + 2 < n ? lower(c[i + 2]) : 0;
        if (a == 's' || a == 't') return i + 2;
        if ((a == 'r' && b == 'e') || (a == 'v' && b == 'e')) return i + 3;
        if (a == 'm') return i + 2;
        if (a == 'l' && b == 'l') return i + 3;
        if (a == 'd') return i + 2;
    }
    // 2. letters, with at most one leading character that is none of CR, LF, letter, number
    {
        size_t j = i;
        if (!is_newline(c0) && !is_letter(c0) && !is_number(c0) && i + 1 < n && is_letter(c[i + 1])) j = i + 1;
        if (is_letter(c[j])) {
            while (j < n && is_letter(c[j])) j++;
            return j;
        }
    }
    // 3. one to max_digits numbers
    if (is_number(c0)) {
        size_t j = i;
        while (j < n && j < i + (size_t)max_digits && is_number(c[j])) j++;
        return j;
    }
    // 4. punctuation and symbols, with an optional leading space and trailing newlines
    {
        auto symbol = [](uint32_t x) { return !is_space(x) && !is_letter(x) && !is_number(x); };
        size_t j = i;
        if (c0 == ' ' && i + 1 < n && symbol(c[i + 1])) j = i + 1;
        if (symbol(c[j])) {
            while (j < n && symbol(c[j])) j++;
            while (j < n && is_newline(c[j])) j++;
            return j;
        }
    }
    // what is left starts a run of whitespace
    size_t e = i;
    while (e < n && is_space(c[e])) e++;
    if (e == i) return i + 1;  // unreachable: every character belongs to one of the classes above
    // 5. whitespace up to and including the last newline of the run
    for (size_t j = e; j > i; j--)
        if (is_newline(c[j - 1])) return j;
    // 6. whitespace not followed by a non-space: the whole run at the end of the text, else all but its last character
    if (e == n) return e;
    if (e - 1 > i) return e - 1;
    // 7. whitespace
    return e;
}

void copy_err(const std::string &e, char *err, size_t errlen) {
    if (err && errlen) snprintf(err, errlen, "%s", e.c_str());
}

bool read_file(const std::string &path, std::string *out, std::string *err) {
    std::ifstream f(path, std::ios::binary);
    if (!f) {
        *err = "cannot open " + path;
        return false;
    }
    std::ostringstream ss;
    ss << f.rdbuf();
    *out = ss.str();
    return true;
}

}  // namespace

std::vector<std::pair<size_t, size_t>> BpeTokenizer::pre_tokenize(const char *text, size_t len, int max_digits) {
    std::vector<std::pair<size_t, size_t>> out;
    const CodePoints c = decode_code_points(text, len);
    for (size_t i = 0; i < c.cp.size();) {
        const size_t j = match_piece(c.cp, i, max_digits);
        out.emplace_back(c.at[i], c.at[j]);
        i = j;
    }
    return out;
}

// GPT-2's bytes_to_unicode (src/tokenizer.rs:19-41): printable Latin-1 bytes stand for themselves,
// the other 68 get U+0100 onwards in byte order
void BpeTokenizer::init_byte_alphabet() {
    uint32_t next = 256;
    for (int b = 0; b < 256; b++) {
        const bool printable = (b >= '!' && b <= '~') || (b >= 0xA1 && b <= 0xAC) || (b >= 0xAE && b <= 0xFF);
        const uint32_t cp = printable ? (uint32_t)b : next++;
        byte_utf8_[b].clear();
        append_utf8(&byte_utf8_[b], cp);
        cp_to_byte_[cp] = (uint8_t)b;
    }
}

std::unique_ptr<BpeTokenizer> BpeTokenizer::from_files(const std::string &vocab_path, const std::string &merges_path,
                                                       std::string *err) {
    std::string vocab_text, merges_text;
    if (!read_file(vocab_path, &vocab_text, err) || !read_file(merges_path, &merges_text, err)) return nullptr;
    std::vector<std::pair<std::string, int64_t>> vocab;
    if (!parse_json_string_to_int_map(vocab_text.data(), vocab_text.size(), &vocab, err)) {
        *err = vocab_path + ": " + *err;
        return nullptr;
    }
    std::unique_ptr<BpeTokenizer> t(new BpeTokenizer());
    for (auto &kv : vocab) {
        if (kv.second < 0 || kv.second > 0xFFFFFFFFLL) {
            *err = vocab_path + ": id of \"" + kv.first + "\" outside u32";
            return nullptr;
        }
        t->encoder_[kv.first] = (uint32_t)kv.second;
    }
    for (const auto &kv : t->encoder_) t->decoder_[kv.second] = kv.first;
    // merges.txt: "left right" per line in rank order; lines that start with '#' (the version header)
    // and empty lines do not count (src/tokenizer.rs:54-66)
    uint32_t rank = 0;
    size_t pos = 0;
    while (pos < merges_text.size()) {
        size_t eol = merges_text.find('\n', pos);
        if (eol == std::string::npos) eol = merges_text.size();
        size_t end = eol;
        if (end > pos && merges_text[end - 1] == '\r') end--;
        if (end > pos && merges_text[pos] != '#') t->ranks_[merges_text.substr(pos, end - pos)] = rank++;
        pos = eol + 1;
    }
    t->init_byte_alphabet();
    return t;
}

namespace {

// The Split patterns of the byte-level BPE family this class implements; they differ in the run of numbers.
const char *const PATTERN_QWEN2 =
    "(?i:'s|'t|'re|'ve|'m|'ll|'d)|[^\\r\\n\\p{L}\\p{N}]?\\p{L}+|\\p{N}| ?[^\\s\\p{L}\\p{N}]+[\\r\\n]*|\\s*[\\r\\n]+|\\s+(?!\\S)|\\s+";
const char *const PATTERN_LLAMA3 =
    "(?i:'s|'t|'re|'ve|'m|'ll|'d)|[^\\r\\n\\p{L}\\p{N}]?\\p{L}+|\\p{N}{1,3}| ?[^\\s\\p{L}\\p{N}]+[\\r\\n]*|\\s*[\\r\\n]+|\\s+(?!\\S)|\\s+";

bool json_flag(const Json &o, const char *key, bool dflt = false) {
    const Json *v = o.get(key);
    return v && v->kind == Json::Bool ? v->b : dflt;
}

const std::string *json_str(const Json &o, const char *key) {
    const Json *v = o.get(key);
    return v && v->kind == Json::Str ? &v->str : nullptr;
}

}  // namespace

std::unique_ptr<BpeTokenizer> BpeTokenizer::from_tokenizer_json(const std::string &path, std::string *err) {
    std::string text;
    if (!read_file(path, &text, err)) return nullptr;
    Json j;
    if (!parse_json(text.data(), text.size(), &j, err)) {
        *err = path + ": " + *err;
        return nullptr;
    }
    auto refuse = [&](const std::string &what) {
        *err = path + ": " + what;
        return nullptr;
    };
    const Json *model = j.get("model");
    if (!model || model->kind != Json::Obj) return refuse("no \"model\" object");
    const std::string *mtype = json_str(*model, "type");
    const Json *vocab = model->get("vocab"), *merges = model->get("merges");
    if ((mtype && *mtype != "BPE") || !vocab || vocab->kind != Json::Obj || !merges || merges->kind != Json::Arr)
        return refuse("model is not a BPE with \"vocab\" and \"merges\"");
    // the SentencePiece-style family (Llama-2, TinyLlama, Mistral) says byte_fallback; the byte-level one does not
    const bool spm = json_flag(*model, "byte_fallback");
    for (const char *key : {"unk_token", "continuing_subword_prefix", "end_of_word_suffix", "dropout"}) {
        const Json *v = model->get(key);
        if (spm && std::string(key) == "unk_token") continue;
        if (v && v->kind != Json::Null && !(v->kind == Json::Str && v->str.empty()))
            return refuse(std::string("BPE option \"") + key + "\" is not supported");
    }
    if (!spm && json_flag(*model, "fuse_unk")) return refuse("BPE fuse_unk without byte_fallback is not supported");
    if (spm && (!json_flag(*model, "fuse_unk") || !json_str(*model, "unk_token")))
        return refuse("BPE byte_fallback is supported with fuse_unk and an unk_token (the Llama-2 family)");
    if (spm && json_flag(*model, "ignore_merges")) return refuse("BPE byte_fallback with ignore_merges is not supported");

    std::unique_ptr<BpeTokenizer> t(new BpeTokenizer());
    t->hf_decode_ = true;
    t->spm_ = spm;
    t->ignore_merges_ = json_flag(*model, "ignore_merges");
    for (const auto &kv : vocab->obj) {
        if (kv.second.kind != Json::Num || kv.second.num < 0 || kv.second.num > 4294967295.0)
            return refuse("vocabulary id of \"" + kv.first + "\" is not a u32");
        t->encoder_[kv.first] = (uint32_t)kv.second.num;
    }
    for (const auto &kv : t->encoder_) t->decoder_[kv.second] = kv.first;
    uint32_t rank = 0;
    for (const Json &m : merges->arr) {  // "left right" strings, or [left, right] pairs
        if (m.kind == Json::Str) {
            t->ranks_[m.str] = rank++;
        } else if (m.kind == Json::Arr && m.arr.size() == 2 && m.arr[0].kind == Json::Str && m.arr[1].kind == Json::Str) {
            t->ranks_[m.arr[0].str + " " + m.arr[1].str] = rank++;
        } else {
            return refuse("merge " + std::to_string(rank) + " is neither a string nor a pair of strings");
        }
    }
    t->init_byte_alphabet();
    if (spm) {
        static const char U2581[] = "\xE2\x96\x81";  // U+2581, the stand-in for a space
        t->unk_id_ = t->token_to_id(*json_str(*model, "unk_token"));
        if (t->unk_id_ < 0) return refuse("unk_token is not in the vocabulary");
        for (int b = 0; b < 256; b++) {
            char name[8];
            snprintf(name, sizeof(name), "<0x%02X>", b);
            t->byte_ids_[b] = t->token_to_id(name);
        }
        // normaliser: Sequence[Prepend(U+2581), Replace(" " -> U+2581)]
        const Json *nz = j.get("normalizer");
        const Json *parts = nz && nz->kind == Json::Obj ? nz->get("normalizers") : nullptr;
        bool ok = nz && nz->kind == Json::Obj && json_str(*nz, "type") && *json_str(*nz, "type") == "Sequence" && parts &&
                  parts->kind == Json::Arr && parts->arr.size() == 2;
        if (ok) {
            const Json &pre = parts->arr[0], &rep = parts->arr[1];
            const Json *pat = rep.kind == Json::Obj ? rep.get("pattern") : nullptr;
            ok = pre.kind == Json::Obj && json_str(pre, "type") && *json_str(pre, "type") == "Prepend" && json_str(pre, "prepend") &&
                 *json_str(pre, "prepend") == U2581 && rep.kind == Json::Obj && json_str(rep, "type") &&
                 *json_str(rep, "type") == "Replace" && pat && pat->kind == Json::Obj && json_str(*pat, "String") &&
                 *json_str(*pat, "String") == " " && json_str(rep, "content") && *json_str(rep, "content") == U2581;
        }
        if (!ok) return refuse("normalizer must be Sequence[Prepend(U+2581), Replace(\" \" -> U+2581)] for a byte_fallback BPE");
        if (const Json *pt = j.get("pre_tokenizer"); pt && pt->kind != Json::Null)
            return refuse("a byte_fallback BPE must have no pre-tokeniser");
        // decoder: Sequence[Replace(U+2581 -> " "), ByteFallback, Fuse, Strip(" ", 1, 0)]
        const Json *dec = j.get("decoder");
        const Json *dparts = dec && dec->kind == Json::Obj ? dec->get("decoders") : nullptr;
        ok = dec && dec->kind == Json::Obj && json_str(*dec, "type") && *json_str(*dec, "type") == "Sequence" && dparts &&
             dparts->kind == Json::Arr && dparts->arr.size() == 4;
        if (ok) {
            const Json &d0 = dparts->arr[0], &d1 = dparts->arr[1], &d2 = dparts->arr[2], &d3 = dparts->arr[3];
            auto type_is = [](const Json &e, const char *name) {
                return e.kind == Json::Obj && json_str(e, "type") && *json_str(e, "type") == name;
            };
            const Json *pat = d0.kind == Json::Obj ? d0.get("pattern") : nullptr;
            const Json *start = d3.kind == Json::Obj ? d3.get("start") : nullptr, *stop = d3.kind == Json::Obj ? d3.get("stop") : nullptr;
            ok = type_is(d0, "Replace") && pat && pat->kind == Json::Obj && json_str(*pat, "String") && *json_str(*pat, "String") == U2581 &&
                 json_str(d0, "content") && *json_str(d0, "content") == " " && type_is(d1, "ByteFallback") && type_is(d2, "Fuse") &&
                 type_is(d3, "Strip") && json_str(d3, "content") && *json_str(d3, "content") == " " && start &&
                 start->kind == Json::Num && start->num == 1 && stop && stop->kind == Json::Num && stop->num == 0;
        }
        if (!ok) return refuse("decoder must be Sequence[Replace(U+2581 -> \" \"), ByteFallback, Fuse, Strip(\" \", 1, 0)] for a byte_fallback BPE");
    }

    // normaliser: none, or NFC (left to the caller)
    if (const Json *nz = j.get("normalizer"); !spm && nz && nz->kind == Json::Obj) {
        const std::string *ty = json_str(*nz, "type");
        if (!ty || *ty != "NFC") return refuse("normalizer " + (ty ? *ty : std::string("?")) + " is not supported (none or NFC)");
        t->wants_nfc_ = true;
    }
    // pre-tokeniser: Sequence[Split(pattern, Isolated), ByteLevel(use_regex = false)]
    if (!spm) {
        const Json *pt = j.get("pre_tokenizer");
        std::vector<const Json *> parts;
        if (pt && pt->kind == Json::Obj) {
            const std::string *ty = json_str(*pt, "type");
            const Json *seq = pt->get("pretokenizers");
            if (ty && *ty == "Sequence" && seq && seq->kind == Json::Arr)
                for (const Json &e : seq->arr) parts.push_back(&e);
            else
                parts.push_back(pt);
        }
        bool have_split = false, have_bytes = false;
        for (const Json *e : parts) {
            const std::string *ty = e->kind == Json::Obj ? json_str(*e, "type") : nullptr;
            if (ty && *ty == "Split") {
                const Json *pat = e->get("pattern");
                const std::string *re = pat && pat->kind == Json::Obj ? json_str(*pat, "Regex") : nullptr;
                const std::string *beh = json_str(*e, "behavior");
                if (!re || !beh || *beh != "Isolated" || json_flag(*e, "invert"))
                    return refuse("Split pre-tokeniser must be an isolated, non-inverted regex");
                if (*re == PATTERN_QWEN2) t->max_digits_ = 1;
                else if (*re == PATTERN_LLAMA3) t->max_digits_ = 3;
                else return refuse("Split pattern is not one of the two this tokenizer implements: " + *re);
                have_split = true;
            } else if (ty && *ty == "ByteLevel") {
                if (json_flag(*e, "add_prefix_space", true)) return refuse("ByteLevel add_prefix_space is not supported");
                if (json_flag(*e, "use_regex", true)) return refuse("ByteLevel with its own (GPT-2) regex is not supported");
                have_bytes = true;
            } else {
                return refuse("pre-tokeniser " + (ty ? *ty : std::string("?")) + " is not supported");
            }
        }
        if (!have_split || !have_bytes) return refuse("pre-tokeniser must be Split + ByteLevel");
    }
    if (const Json *dec = j.get("decoder"); !spm && (!dec || dec->kind != Json::Obj || !json_str(*dec, "type") || *json_str(*dec, "type") != "ByteLevel"))
        return refuse("decoder must be ByteLevel");

    // added tokens
    if (const Json *added = j.get("added_tokens"); added && added->kind == Json::Arr) {
        for (const Json &a : added->arr) {
            const Json *id = a.kind == Json::Obj ? a.get("id") : nullptr;
            const std::string *content = a.kind == Json::Obj ? json_str(a, "content") : nullptr;
            if (!id || id->kind != Json::Num || !content || content->empty()) return refuse("malformed added token");
            if (json_flag(a, "lstrip") || json_flag(a, "rstrip") || json_flag(a, "single_word"))
                return refuse("added token \"" + *content + "\": lstrip / rstrip / single_word are not supported");
            if (spm && json_flag(a, "normalized"))
                return refuse("added token \"" + *content + "\": normalized added tokens are not supported with a byte_fallback BPE");
            t->added_.push_back(Added{*content, (uint32_t)id->num, json_flag(a, "special")});
        }
        std::stable_sort(t->added_.begin(), t->added_.end(),
                         [](const Added &x, const Added &y) { return x.content.size() > y.content.size(); });
        for (size_t i = 0; i < t->added_.size(); i++) {
            t->added_by_id_[t->added_[i].id] = i;
            t->decoder_[t->added_[i].id] = t->added_[i].content;
        }
    }
    // post-processor: ByteLevel changes no ids; TemplateProcessing wraps a single sequence in special tokens
    if (const Json *pp = j.get("post_processor"); pp && pp->kind == Json::Obj) {
        std::vector<const Json *> parts;
        const std::string *ty = json_str(*pp, "type");
        const Json *seq = pp->get("processors");
        if (ty && *ty == "Sequence" && seq && seq->kind == Json::Arr)
            for (const Json &e : seq->arr) parts.push_back(&e);
        else
            parts.push_back(pp);
        for (const Json *e : parts) {
            const std::string *pty = e->kind == Json::Obj ? json_str(*e, "type") : nullptr;
            if (pty && *pty == "ByteLevel") continue;
            if (!pty || *pty != "TemplateProcessing") return refuse("post-processor " + (pty ? *pty : std::string("?")) + " is not supported");
            const Json *single = e->get("single");
            if (!single || single->kind != Json::Arr) return refuse("TemplateProcessing without \"single\"");
            bool seen_a = false;
            for (const Json &item : single->arr) {
                if (item.kind != Json::Obj) return refuse("malformed TemplateProcessing item");
                if (const Json *sp = item.get("SpecialToken"); sp && sp->kind == Json::Obj) {
                    const std::string *name = json_str(*sp, "id");
                    const int64_t id = name ? t->token_to_id(*name) : -1;
                    if (id < 0) return refuse("TemplateProcessing names an unknown special token");
                    (seen_a ? t->suffix_ids_ : t->prefix_ids_).push_back((uint32_t)id);
                } else if (item.get("Sequence")) {
                    seen_a = true;
                }
            }
        }
    }
    return t;
}

int64_t BpeTokenizer::token_to_id(const std::string &token) const {
    for (const Added &a : added_)
        if (a.content == token) return a.id;
    auto it = encoder_.find(token);
    return it == encoder_.end() ? -1 : (int64_t)it->second;
}

// reference bpe (src/tokenizer.rs:85-116): while some adjacent pair has a rank, merge the first
// occurrence of the pair with the lowest rank
std::vector<std::string> BpeTokenizer::bpe(const std::string &mapped) const {
    std::vector<std::string> word;
    for (size_t i = 0; i < mapped.size();) {
        uint32_t cp;
        size_t bad;
        const size_t n = utf8_at(reinterpret_cast<const unsigned char *>(mapped.data()) + i, mapped.size() - i, &cp, &bad);
        word.emplace_back(mapped, i, n ? n : 1);
        i += n ? n : 1;
    }
    while (word.size() > 1) {
        size_t best = word.size();
        uint32_t best_rank = 0xFFFFFFFFu;
        std::string key;
        for (size_t i = 0; i + 1 < word.size(); i++) {
            key.assign(word[i]);
            key.push_back(' ');
            key.append(word[i + 1]);
            auto it = ranks_.find(key);
            if (it != ranks_.end() && it->second < best_rank) {
                best_rank = it->second;
                best = i;
            }
        }
        if (best == word.size()) break;
        word[best] += word[best + 1];
        word.erase(word.begin() + (long)best + 1);
    }
    return word;
}

// The SentencePiece-style family as the `tokenizers` crate runs it (models/bpe: merge_word and Word::merge_all):
// the normalised stretch - U+2581 in front, spaces replaced by U+2581 - is one word; a character that is a
// vocabulary entry is a symbol, any other goes in as its UTF-8 bytes "<0xXX>" (or as the unknown token, runs of
// which are fused, when a byte token is missing); then the adjacent pair with the lowest merge rank, leftmost
// among equals, is merged until none is left. A heap of candidate pairs keeps this near-linear for long texts.
void BpeTokenizer::encode_plain_spm(const char *text, size_t len, std::vector<uint32_t> *ids) const {
    if (len == 0) return;
    static const char U2581[] = "\xE2\x96\x81";
    std::string norm(U2581);
    for (size_t i = 0; i < len; i++) {
        if (text[i] == ' ') norm += U2581;
        else norm.push_back(text[i]);
    }
    struct Sym {
        std::string s;
        int64_t id;  // vocabulary id; merges look the strings up
        int prev, next;
        uint32_t ver;
        bool alive;
    };
    std::vector<Sym> w;
    auto push = [&](std::string str, int64_t id) {
        Sym y{std::move(str), id, (int)w.size() - 1, -1, 0, true};
        if (!w.empty()) w.back().next = (int)w.size();
        w.push_back(std::move(y));
    };
    // An unknown character waits (fuse_unk: a run of them is one unknown token) until the next vocabulary character or
    // the end of the word puts it in; byte tokens in between do not, exactly as the crate's merge_word has it.
    bool unk_waits = false;
    auto put_unk = [&]() {
        if (unk_waits) push(decoder_.at((uint32_t)unk_id_), unk_id_);
        unk_waits = false;
    };
    for (size_t i = 0; i < norm.size();) {
        uint32_t cp;
        size_t bad;
        size_t n = utf8_at(reinterpret_cast<const unsigned char *>(norm.data()) + i, norm.size() - i, &cp, &bad);
        if (!n) n = 1;  // ill-formed input: byte by byte (the caller hands valid UTF-8)
        std::string ch(norm, i, n);
        i += n;
        auto it = encoder_.find(ch);
        if (it != encoder_.end()) {
            put_unk();
            push(std::move(ch), it->second);
            continue;
        }
        bool all = true;
        for (unsigned char b : ch) all = all && byte_ids_[b] >= 0;
        if (all) {
            for (unsigned char b : ch) {
                char name[8];
                snprintf(name, sizeof(name), "<0x%02X>", (unsigned)b);
                push(name, byte_ids_[b]);
            }
        } else {
            unk_waits = true;
        }
    }
    put_unk();
    struct Cand {
        uint32_t rank;
        int left, right;
        uint32_t lver, rver;
    };
    auto worse = [](const Cand &a, const Cand &b) { return a.rank != b.rank ? a.rank > b.rank : a.left > b.left; };
    std::priority_queue<Cand, std::vector<Cand>, decltype(worse)> heap(worse);
    std::string key;
    auto offer = [&](int l) {
        if (l < 0 || w[l].next < 0) return;
        const int r = w[l].next;
        key.assign(w[l].s);
        key.push_back(' ');
        key.append(w[r].s);
        auto it = ranks_.find(key);
        if (it != ranks_.end()) heap.push(Cand{it->second, l, r, w[l].ver, w[r].ver});
    };
    for (int i = 0; i + 1 < (int)w.size(); i++) offer(i);
    while (!heap.empty()) {
        const Cand c = heap.top();
        heap.pop();
        Sym &l = w[c.left], &r = w[c.right];
        if (!l.alive || !r.alive || l.ver != c.lver || r.ver != c.rver || l.next != c.right) continue;  // a stale pair
        l.s += r.s;
        auto id = encoder_.find(l.s);
        l.id = id == encoder_.end() ? -1 : (int64_t)id->second;
        l.ver++;
        r.alive = false;
        l.next = r.next;
        if (r.next >= 0) w[r.next].prev = c.left;
        offer(l.prev);
        offer(c.left);
    }
    for (int i = w.empty() ? -1 : 0; i >= 0; i = w[i].next)
        if (w[i].id >= 0) ids->push_back((uint32_t)w[i].id);
}

// Decoder of that family: U+2581 back to spaces, runs of byte tokens to the text they spell (every byte of a run
// that is not UTF-8 becomes U+FFFD), everything joined, one leading space dropped.
std::string BpeTokenizer::decode_spm(const uint32_t *ids, size_t n, bool skip_special) const {
    static const char U2581[] = "\xE2\x96\x81";
    std::string out, run;
    auto flush = [&]() {
        if (run.empty()) return;
        bool valid = true;
        for (size_t i = 0; i < run.size() && valid;) {
            uint32_t cp;
            size_t bad;
            const size_t m = utf8_at(reinterpret_cast<const unsigned char *>(run.data()) + i, run.size() - i, &cp, &bad);
            valid = m != 0;
            i += m ? m : 1;
        }
        if (valid) out += run;
        else
            for (size_t i = 0; i < run.size(); i++) out += "\xEF\xBF\xBD";
        run.clear();
    };
    for (size_t k = 0; k < n; k++) {
        auto it = decoder_.find(ids[k]);
        if (it == decoder_.end()) continue;
        if (skip_special) {
            auto a = added_by_id_.find(ids[k]);
            if (a != added_by_id_.end() && added_[a->second].special) continue;
        }
        const std::string &tok = it->second;
        unsigned byte = 0;
        if (tok.size() == 6 && tok.compare(0, 3, "<0x") == 0 && tok[5] == '>' && isxdigit((unsigned char)tok[3]) &&
            isxdigit((unsigned char)tok[4]) && sscanf(tok.c_str() + 3, "%2x", &byte) == 1) {
            run.push_back((char)byte);
            continue;
        }
        flush();
        for (size_t i = 0; i < tok.size();) {
            if (tok.compare(i, 3, U2581) == 0) {
                out.push_back(' ');
                i += 3;
            } else {
                out.push_back(tok[i++]);
            }
        }
    }
    flush();
    if (!out.empty() && out[0] == ' ') out.erase(0, 1);
    return out;
}

void BpeTokenizer::encode_plain(const char *text, size_t len, std::vector<uint32_t> *ids) const {
    if (spm_) {
        encode_plain_spm(text, len, ids);
        return;
    }
    std::string mapped;
    for (const auto &piece : pre_tokenize(text, len, max_digits_)) {
        mapped.clear();
        for (size_t i = piece.first; i < piece.second; i++) mapped += byte_utf8_[(unsigned char)text[i]];
        if (ignore_merges_) {
            auto whole = encoder_.find(mapped);
            if (whole != encoder_.end()) {
                ids->push_back(whole->second);
                continue;
            }
        }
        for (const std::string &sym : bpe(mapped)) {
            auto it = encoder_.find(sym);
            if (it != encoder_.end()) ids->push_back(it->second);
        }
    }
}

std::vector<uint32_t> BpeTokenizer::encode(const char *text, size_t len, bool add_special_tokens) const {
    std::vector<uint32_t> ids;
    if (add_special_tokens) ids = prefix_ids_;
    if (added_.empty()) {
        encode_plain(text, len, &ids);
    } else {
        // added tokens stand for themselves: the leftmost match wins, the longest at that position
        // (added_ is sorted by length); the stretches between them are ordinary text
        size_t plain_from = 0;
        for (size_t i = 0; i < len;) {
            const Added *hit = nullptr;
            for (const Added &a : added_) {
                if (a.content.size() <= len - i && text[i] == a.content[0] && memcmp(text + i, a.content.data(), a.content.size()) == 0) {
                    hit = &a;
                    break;
                }
            }
            if (!hit) {
                i++;
                continue;
            }
            if (i > plain_from) encode_plain(text + plain_from, i - plain_from, &ids);
            ids.push_back(hit->id);
            i += hit->content.size();
            plain_from = i;
        }
        if (len > plain_from) encode_plain(text + plain_from, len - plain_from, &ids);
    }
    if (add_special_tokens) ids.insert(ids.end(), suffix_ids_.begin(), suffix_ids_.end());
    return ids;
}

std::string BpeTokenizer::decode(const uint32_t *ids, size_t n, bool skip_special) const {
    if (spm_) return decode_spm(ids, n, skip_special);
    std::string bytes, tok_bytes;
    for (size_t k = 0; k < n; k++) {
        auto it = decoder_.find(ids[k]);
        if (it == decoder_.end()) continue;
        if (skip_special) {
            auto a = added_by_id_.find(ids[k]);
            if (a != added_by_id_.end() && added_[a->second].special) continue;
        }
        const std::string &tok = it->second;
        tok_bytes.clear();
        bool all_mapped = true;
        for (size_t i = 0; i < tok.size();) {
            uint32_t cp;
            size_t bad;
            const size_t m = utf8_at(reinterpret_cast<const unsigned char *>(tok.data()) + i, tok.size() - i, &cp, &bad);
            if (m) {
                auto b = cp_to_byte_.find(cp);
                if (b != cp_to_byte_.end()) tok_bytes.push_back((char)b->second);
                else all_mapped = false;
            } else {
                all_mapped = false;
            }
            i += m ? m : 1;
        }
        // tokenizer.json files: a token with a character outside the byte alphabet is taken as written
        bytes += (hf_decode_ && !all_mapped) ? tok : tok_bytes;
    }
    // String::from_utf8_lossy: every longest ill-formed prefix becomes one U+FFFD
    std::string out;
    const unsigned char *s = reinterpret_cast<const unsigned char *>(bytes.data());
    for (size_t i = 0; i < bytes.size();) {
        uint32_t cp;
        size_t bad;
        const size_t m = utf8_at(s + i, bytes.size() - i, &cp, &bad);
        if (m) {
            out.append(bytes, i, m);
            i += m;
        } else {
            out += "\xEF\xBF\xBD";
            i += bad;
        }
    }
    return out;
}

}  // namespace homura

struct hm_tokenizer {
    std::unique_ptr<homura::BpeTokenizer> t;
};

#pragma GCC visibility push(default)
extern "C" {

hm_tokenizer *hm_tokenizer_open(const char *vocab_json_path, const char *merges_txt_path, char *err, size_t errlen) {
    std::string e;
    auto t = homura::BpeTokenizer::from_files(vocab_json_path ? vocab_json_path : "", merges_txt_path ? merges_txt_path : "", &e);
    if (!t) {
        homura::copy_err(e, err, errlen);
        return nullptr;
    }
    return new hm_tokenizer{std::move(t)};
}

hm_tokenizer *hm_tokenizer_open_json(const char *tokenizer_json_path, char *err, size_t errlen) {
    std::string e;
    auto t = homura::BpeTokenizer::from_tokenizer_json(tokenizer_json_path ? tokenizer_json_path : "", &e);
    if (!t) {
        homura::copy_err(e, err, errlen);
        return nullptr;
    }
    return new hm_tokenizer{std::move(t)};
}

void hm_tokenizer_close(hm_tokenizer *t) { delete t; }

int hm_tokenizer_wants_nfc(const hm_tokenizer *t) { return t ? (t->t->wants_nfc() ? 1 : 0) : HM_ERR_INVALID; }

long long hm_tokenizer_token_to_id(const hm_tokenizer *t, const char *token) {
    if (!t || !token) return -1;
    return (long long)t->t->token_to_id(token);
}

long long hm_tokenizer_encode_ex(const hm_tokenizer *t, const char *text, size_t text_len, int add_special_tokens,
                                 uint32_t *ids_out, size_t capacity) {
    if (!t || (!text && text_len) || (!ids_out && capacity)) return HM_ERR_INVALID;
    const std::vector<uint32_t> ids = t->t->encode(text, text_len, add_special_tokens != 0);
    const size_t n = std::min(ids.size(), capacity);
    if (n) memcpy(ids_out, ids.data(), n * sizeof(uint32_t));
    return (long long)ids.size();
}

long long hm_tokenizer_decode_ex(const hm_tokenizer *t, const uint32_t *ids, size_t n_ids, int skip_special_tokens,
                                 char *text_out, size_t capacity) {
    if (!t || (!ids && n_ids) || (!text_out && capacity)) return HM_ERR_INVALID;
    const std::string s = t->t->decode(ids, n_ids, skip_special_tokens != 0);
    const size_t n = std::min(s.size(), capacity);
    if (n) memcpy(text_out, s.data(), n);
    return (long long)s.size();
}

int hm_tokenizer_vocab_size(const hm_tokenizer *t) { return t ? (int)t->t->vocab_size() : HM_ERR_INVALID; }

long long hm_tokenizer_encode(const hm_tokenizer *t, const char *text, size_t text_len, uint32_t *ids_out, size_t capacity) {
    if (!t || (!text && text_len) || (!ids_out && capacity)) return HM_ERR_INVALID;
    const std::vector<uint32_t> ids = t->t->encode(text, text_len);
    const size_t n = std::min(ids.size(), capacity);
    if (n) memcpy(ids_out, ids.data(), n * sizeof(uint32_t));
    return (long long)ids.size();
}

long long hm_tokenizer_decode(const hm_tokenizer *t, const uint32_t *ids, size_t n_ids, char *text_out, size_t capacity) {
    if (!t || (!ids && n_ids) || (!text_out && capacity)) return HM_ERR_INVALID;
    const std::string s = t->t->decode(ids, n_ids);
    const size_t n = std::min(s.size(), capacity);
    if (n) memcpy(text_out, s.data(), n);
    return (long long)s.size();
}

long long hm_tokenizer_pieces(const char *text, size_t text_len, size_t *ends_out, size_t capacity) {
    if ((!text && text_len) || (!ends_out && capacity)) return HM_ERR_INVALID;
    const auto pieces = homura::BpeTokenizer::pre_tokenize(text, text_len);
    for (size_t i = 0; i < pieces.size() && i < capacity; i++) ends_out[i] = pieces[i].second;
    return (long long)pieces.size();
}

}  // extern "C"
#pragma GCC visibility pop
