// The one JSON shape the tokenizer needs, read by the JSON parser of loaders.hip.
#pragma once

#include <cstdint>
#include <string>
#include <utility>
#include <vector>

namespace homura {

// A JSON object whose values are all integers (vocab.json: token -> id), in file order.
bool parse_json_string_to_int_map(const char *text, size_t len, std::vector<std::pair<std::string, int64_t>> *out,
                                  std::string *err);

}  // namespace homura
