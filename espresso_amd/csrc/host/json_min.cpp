#include "json_min.h"

#include <cctype>
#include <cstdlib>

namespace esp {
namespace {

struct Cursor {
    const std::string &s;
    size_t i = 0;
    std::string err;
    void ws() { while (i < s.size() && std::isspace((unsigned char)s[i])) i++; }
    bool eat(char c) { ws(); if (i < s.size() && s[i] == c) { i++; return true; } return false; }
    bool fail(const std::string &m) { if (err.empty()) err = m + " at offset " + std::to_string(i); return false; }
};

bool parse_string(Cursor &c, std::string *out) {
    c.ws();
    if (c.i >= c.s.size() || c.s[c.i] != '"') return c.fail("expected string");
    c.i++;
    out->clear();
    while (c.i < c.s.size() && c.s[c.i] != '"') {
        char ch = c.s[c.i++];
        if (ch == '\\') {
            if (c.i >= c.s.size()) return c.fail("bad escape");
            char e = c.s[c.i++];
            switch (e) {
            case 'n': out->push_back('\n'); break;
            case 't': out->push_back('\t'); break;
            case 'r': out->push_back('\r'); break;
            case 'b': out->push_back('\b'); break;
            case 'f': out->push_back('\f'); break;
            case 'u': {
                if (c.i + 4 > c.s.size()) return c.fail("bad \\u escape");
                unsigned cp = (unsigned)std::strtoul(c.s.substr(c.i, 4).c_str(), nullptr, 16);
                c.i += 4;
                // a high surrogate followed by an escaped low surrogate is one code point
                if (cp >= 0xD800 && cp < 0xDC00 && c.i + 6 <= c.s.size() && c.s[c.i] == '\\' && c.s[c.i + 1] == 'u') {
                    const unsigned lo = (unsigned)std::strtoul(c.s.substr(c.i + 2, 4).c_str(), nullptr, 16);
                    if (lo >= 0xDC00 && lo < 0xE000) { cp = 0x10000 + ((cp - 0xD800) << 10) + (lo - 0xDC00); c.i += 6; }
                }
                if (cp >= 0xD800 && cp < 0xE000) cp = 0xFFFD;   // lone surrogate
                if (cp < 0x80) out->push_back((char)cp);
                else if (cp < 0x800) { out->push_back((char)(0xC0 | (cp >> 6))); out->push_back((char)(0x80 | (cp & 0x3F))); }
                else if (cp < 0x10000) { out->push_back((char)(0xE0 | (cp >> 12))); out->push_back((char)(0x80 | ((cp >> 6) & 0x3F))); out->push_back((char)(0x80 | (cp & 0x3F))); }
                else { out->push_back((char)(0xF0 | (cp >> 18))); out->push_back((char)(0x80 | ((cp >> 12) & 0x3F))); out->push_back((char)(0x80 | ((cp >> 6) & 0x3F))); out->push_back((char)(0x80 | (cp & 0x3F))); }
                break;
            }
            default: out->push_back(e);
            }
        } else out->push_back(ch);
    }
    if (c.i >= c.s.size()) return c.fail("unterminated string");
    c.i++;
    return true;
}

bool skip_value(Cursor &c);

bool skip_container(Cursor &c, char open, char close) {
    if (!c.eat(open)) return c.fail("expected container");
    if (c.eat(close)) return true;
    for (;;) {
        if (open == '{') {
            std::string k;
            if (!parse_string(c, &k) || !c.eat(':')) return c.fail("bad object member");
        }
        if (!skip_value(c)) return false;
        if (c.eat(close)) return true;
        if (!c.eat(',')) return c.fail("expected , or closing bracket");
    }
}

bool parse_scalar(Cursor &c, JsonValue *v) {
    c.ws();
    if (c.i >= c.s.size()) return c.fail("unexpected end");
    char ch = c.s[c.i];
    if (ch == '"') { v->kind = JsonValue::String; return parse_string(c, &v->text); }
    if (c.s.compare(c.i, 4, "true") == 0) { c.i += 4; v->kind = JsonValue::Bool; v->boolean = true; return true; }
    if (c.s.compare(c.i, 5, "false") == 0) { c.i += 5; v->kind = JsonValue::Bool; v->boolean = false; return true; }
    if (c.s.compare(c.i, 4, "null") == 0) { c.i += 4; v->kind = JsonValue::Null; return true; }
    if (ch == '{') { v->kind = JsonValue::Other; return skip_container(c, '{', '}'); }
    if (ch == '[') { v->kind = JsonValue::Other; return skip_container(c, '[', ']'); }
    char *end = nullptr;
    double d = std::strtod(c.s.c_str() + c.i, &end);
    if (end == c.s.c_str() + c.i) return c.fail("unexpected character");
    c.i = (size_t)(end - c.s.c_str());
    v->kind = JsonValue::Number;
    v->number = d;
    return true;
}

bool skip_value(Cursor &c) { JsonValue v; return parse_scalar(c, &v); }

bool parse_node(Cursor &c, JsonNode *n, int depth) {
    if (depth > 64) return c.fail("nesting too deep");
    c.ws();
    if (c.i >= c.s.size()) return c.fail("unexpected end");
    const char ch = c.s[c.i];
    if (ch == '{') {
        c.i++;
        n->kind = JsonNode::Object;
        if (c.eat('}')) return true;
        for (;;) {
            std::string key;
            if (!parse_string(c, &key)) return false;
            if (!c.eat(':')) return c.fail("expected :");
            n->members.emplace_back(std::move(key), JsonNode{});
            if (!parse_node(c, &n->members.back().second, depth + 1)) return false;
            if (c.eat('}')) return true;
            if (!c.eat(',')) return c.fail("expected , or }");
        }
    }
    if (ch == '[') {
        c.i++;
        n->kind = JsonNode::Array;
        if (c.eat(']')) return true;
        for (;;) {
            n->items.emplace_back();
            if (!parse_node(c, &n->items.back(), depth + 1)) return false;
            if (c.eat(']')) return true;
            if (!c.eat(',')) return c.fail("expected , or ]");
        }
    }
    JsonValue v;
    if (!parse_scalar(c, &v)) return false;
    switch (v.kind) {
    case JsonValue::Bool: n->kind = JsonNode::Bool; n->boolean = v.boolean; break;
    case JsonValue::Number: n->kind = JsonNode::Number; n->number = v.number; break;
    case JsonValue::String: n->kind = JsonNode::String; n->text = std::move(v.text); break;
    default: n->kind = JsonNode::Null; break;
    }
    return true;
}

}  // namespace

const JsonNode *JsonNode::find(const std::string &key) const {
    const JsonNode *hit = nullptr;
    for (const auto &m : members)
        if (m.first == key) hit = &m.second;
    return hit;
}

bool json_parse(const std::string &text, JsonNode *out, std::string *error) {
    Cursor c{text};
    *out = JsonNode{};
    bool ok = parse_node(c, out, 0);
    if (ok) { c.ws(); if (c.i != text.size()) ok = c.fail("trailing characters"); }
    if (!ok && error) *error = c.err;
    return ok;
}

bool json_parse_object(const std::string &text, JsonObject *out, std::string *error) {
    Cursor c{text};
    out->clear();
    bool ok = [&]() {
        if (!c.eat('{')) return c.fail("expected {");
        if (c.eat('}')) return true;
        for (;;) {
            std::string key;
            if (!parse_string(c, &key)) return false;
            if (!c.eat(':')) return c.fail("expected :");
            JsonValue v;
            if (!parse_scalar(c, &v)) return false;
            (*out)[key] = v;
            if (c.eat('}')) return true;
            if (!c.eat(',')) return c.fail("expected , or }");
        }
    }();
    if (ok) { c.ws(); if (c.i != text.size()) ok = c.fail("trailing characters"); }
    if (!ok && error) *error = c.err;
    return ok;
}

std::string json_escape(const std::string &s) {
    std::string o;
    for (char ch : s) {
        switch (ch) {
        case '"': o += "\\\""; break;
        case '\\': o += "\\\\"; break;
        case '\n': o += "\\n"; break;
        case '\t': o += "\\t"; break;
        case '\r': o += "\\r"; break;
        default: o.push_back(ch);
        }
    }
    return o;
}

}  // namespace esp
