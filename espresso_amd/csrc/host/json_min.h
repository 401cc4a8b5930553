// A minimal JSON reader/writer.  json_parse_object reads the flat objects this library exchanges with
// the reference's tooling (metadata.json, draft descriptors): objects of strings, numbers, booleans and
// null, nested arrays/objects skipped.  json_parse builds the whole tree (tokenizer.json, vocab.json).
#pragma once

#include <map>
#include <string>
#include <utility>
#include <vector>

namespace esp {

struct JsonValue {
    enum Kind { Null, Bool, Number, String, Other } kind = Null;
    double number = 0;
    bool boolean = false;
    std::string text;
};

using JsonObject = std::map<std::string, JsonValue>;

// Returns false (and sets *error) unless `text` is one JSON object.
bool json_parse_object(const std::string &text, JsonObject *out, std::string *error);
std::string json_escape(const std::string &s);

struct JsonNode {
    enum Kind { Null, Bool, Number, String, Array, Object } kind = Null;
    double number = 0;
    bool boolean = false;
    std::string text;                                          // String, UTF-8
    std::vector<JsonNode> items;                               // Array
    std::vector<std::pair<std::string, JsonNode>> members;     // Object, in file order
    // the last member named `key` (a later duplicate replaces an earlier one), or nullptr
    const JsonNode *find(const std::string &key) const;
    bool is(Kind k) const { return kind == k; }
};
// Returns false (and sets *error) unless `text` is one JSON value.
bool json_parse(const std::string &text, JsonNode *out, std::string *error);

}  // namespace esp
