// A minimal JSON reader/writer for the flat objects this library exchanges with the reference's
// tooling (metadata.json, draft descriptors): objects of strings, numbers, booleans and null.
// Nested arrays/objects are skipped on read.
#pragma once

#include <map>
#include <string>

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

}  // namespace esp
