// A small JSON reader: config.json, safetensors headers, shard indices, tokenizer.json.
// Plain C++ (no device headers), so host-only translation units can use it too.
#pragma once

#include <cstdint>
#include <cstdlib>
#include <cstring>
#include <string>
#include <utility>
#include <vector>

namespace homura {

struct Json {
    enum Kind { Null, Bool, Num, Str, Arr, Obj } kind = Null;
    bool b = false;
    double num = 0;
    std::string str;
    std::vector<Json> arr;
    std::vector<std::pair<std::string, Json>> obj;
    const Json *get(const std::string &key) const {
        if (kind != Obj) return nullptr;
        for (const auto &kv : obj)
            if (kv.first == key) return &kv.second;
        return nullptr;
    }
};

struct JsonParser {
    const char *p, *end;
    std::string err;
    int depth = 0;
    void ws() {
        while (p < end && (*p == ' ' || *p == '\t' || *p == '\n' || *p == '\r')) p++;
    }
    bool fail(const char *what) {
        if (err.empty()) err = std::string("JSON: ") + what;
        return false;
    }
    bool string(std::string *out) {
        if (p >= end || *p != '"') return fail("expected a string");
        p++;
        out->clear();
        while (p < end && *p != '"') {
            if (*p == '\\') {
                if (++p >= end) return fail("unterminated escape");
                switch (*p) {
                case '"': out->push_back('"'); break;
                case '\\': out->push_back('\\'); break;
                case '/': out->push_back('/'); break;
                case 'b': out->push_back('\b'); break;
                case 'f': out->push_back('\f'); break;
                case 'n': out->push_back('\n'); break;
                case 'r': out->push_back('\r'); break;
                case 't': out->push_back('\t'); break;
                case 'u': {
                    if (end - p < 5) return fail("short \\u escape");
                    unsigned cp = 0;
                    for (int i = 1; i <= 4; i++) {
                        const char ch = p[i];
                        cp <<= 4;
                        if (ch >= '0' && ch <= '9') cp |= ch - '0';
                        else if (ch >= 'a' && ch <= 'f') cp |= ch - 'a' + 10;
                        else if (ch >= 'A' && ch <= 'F') cp |= ch - 'A' + 10;
                        else return fail("bad \\u escape");
                    }
                    p += 4;
                    if (cp >= 0xD800 && cp < 0xDC00 && end - p >= 7 && p[1] == '\\' && p[2] == 'u') {  // surrogate pair
                        unsigned lo = 0;
                        bool hex = true;
                        for (int i = 3; i <= 6; i++) {
                            const char ch = p[i];
                            lo <<= 4;
                            if (ch >= '0' && ch <= '9') lo |= ch - '0';
                            else if (ch >= 'a' && ch <= 'f') lo |= ch - 'a' + 10;
                            else if (ch >= 'A' && ch <= 'F') lo |= ch - 'A' + 10;
                            else hex = false;
                        }
                        if (hex && lo >= 0xDC00 && lo < 0xE000) {
                            cp = 0x10000 + ((cp - 0xD800) << 10) + (lo - 0xDC00);
                            p += 6;
                        }
                    }
                    if (cp >= 0x10000) {
                        out->push_back((char)(0xF0 | (cp >> 18)));
                        out->push_back((char)(0x80 | ((cp >> 12) & 0x3F)));
                        out->push_back((char)(0x80 | ((cp >> 6) & 0x3F)));
                        out->push_back((char)(0x80 | (cp & 0x3F)));
                    } else if (cp < 0x80) {
                        out->push_back((char)cp);
                    } else if (cp < 0x800) {
                        out->push_back((char)(0xC0 | (cp >> 6)));
                        out->push_back((char)(0x80 | (cp & 0x3F)));
                    } else {
                        out->push_back((char)(0xE0 | (cp >> 12)));
                        out->push_back((char)(0x80 | ((cp >> 6) & 0x3F)));
                        out->push_back((char)(0x80 | (cp & 0x3F)));
                    }
                    break;
                }
                default: return fail("unknown escape");
                }
                p++;
            } else {
                out->push_back(*p++);
            }
        }
        if (p >= end) return fail("unterminated string");
        p++;
        return true;
    }
    bool value(Json *v) {
        if (++depth > 64) return fail("nesting too deep");
        ws();
        if (p >= end) return fail("unexpected end");
        bool ok = true;
        if (*p == '{') {
            v->kind = Json::Obj;
            p++;
            ws();
            if (p < end && *p == '}') {
                p++;
            } else {
                for (;;) {
                    ws();
                    std::string key;
                    if (!string(&key)) return false;
                    ws();
                    if (p >= end || *p != ':') return fail("expected ':'");
                    p++;
                    v->obj.emplace_back(std::move(key), Json());
                    if (!value(&v->obj.back().second)) return false;
                    ws();
                    if (p < end && *p == ',') { p++; continue; }
                    if (p < end && *p == '}') { p++; break; }
                    return fail("expected ',' or '}'");
                }
            }
        } else if (*p == '[') {
            v->kind = Json::Arr;
            p++;
            ws();
            if (p < end && *p == ']') {
                p++;
            } else {
                for (;;) {
                    v->arr.emplace_back();
                    if (!value(&v->arr.back())) return false;
                    ws();
                    if (p < end && *p == ',') { p++; continue; }
                    if (p < end && *p == ']') { p++; break; }
                    return fail("expected ',' or ']'");
                }
            }
        } else if (*p == '"') {
            v->kind = Json::Str;
            ok = string(&v->str);
        } else if (end - p >= 4 && std::strncmp(p, "true", 4) == 0) {
            v->kind = Json::Bool; v->b = true; p += 4;
        } else if (end - p >= 5 && std::strncmp(p, "false", 5) == 0) {
            v->kind = Json::Bool; v->b = false; p += 5;
        } else if (end - p >= 4 && std::strncmp(p, "null", 4) == 0) {
            v->kind = Json::Null; p += 4;
        } else {
            const char *q = p;
            while (q < end && (std::strchr("+-.eE", *q) || (*q >= '0' && *q <= '9'))) q++;
            if (q == p) return fail("unexpected character");
            const std::string num(p, q);
            char *stop = nullptr;
            v->num = std::strtod(num.c_str(), &stop);
            if (!stop || *stop) return fail("bad number");
            v->kind = Json::Num;
            p = q;
        }
        depth--;
        return ok;
    }
};

inline bool parse_json(const char *text, size_t len, Json *out, std::string *err) {
    JsonParser jp{text, text + len};
    if (!jp.value(out)) {
        *err = jp.err;
        return false;
    }
    jp.ws();
    if (jp.p != jp.end) {
        *err = "JSON: trailing characters";
        return false;
    }
    return true;
}

// A JSON object whose values are all integers (vocab.json: token -> id), in file order.
bool parse_json_string_to_int_map(const char *text, size_t len, std::vector<std::pair<std::string, int64_t>> *out,
                                  std::string *err);

}  // namespace homura
