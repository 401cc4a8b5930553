#include "regex_min.h"

#include <functional>

#include "unicode_tables.h"

namespace esp {

// ---- UTF-8 ------------------------------------------------------------------------------------------

namespace {

// Decodes one scalar at s[i].  Returns the bytes consumed; *ok is false when they form a maximal
// invalid subpart (to be replaced by U+FFFD).
size_t decode_one(const std::string &s, size_t i, uint32_t *cp, bool *ok) {
    const auto byte = [&](size_t k) -> unsigned { return k < s.size() ? (unsigned char)s[k] : 0x100u; };
    const unsigned b0 = byte(i);
    *ok = true;
    if (b0 < 0x80) { *cp = b0; return 1; }
    int need = 0;
    unsigned lo = 0x80, hi = 0xBF;
    uint32_t v = 0;
    if (b0 >= 0xC2 && b0 <= 0xDF) { need = 1; v = b0 & 0x1F; }
    else if (b0 == 0xE0) { need = 2; v = b0 & 0x0F; lo = 0xA0; }
    else if ((b0 >= 0xE1 && b0 <= 0xEC) || b0 == 0xEE || b0 == 0xEF) { need = 2; v = b0 & 0x0F; }
    else if (b0 == 0xED) { need = 2; v = b0 & 0x0F; hi = 0x9F; }
    else if (b0 == 0xF0) { need = 3; v = b0 & 0x07; lo = 0x90; }
    else if (b0 >= 0xF1 && b0 <= 0xF3) { need = 3; v = b0 & 0x07; }
    else if (b0 == 0xF4) { need = 3; v = b0 & 0x07; hi = 0x8F; }
    else { *ok = false; *cp = 0xFFFD; return 1; }
    size_t used = 1;
    for (int k = 0; k < need; k++) {
        const unsigned b = byte(i + used);
        if (b < lo || b > hi) { *ok = false; *cp = 0xFFFD; return used; }
        v = (v << 6) | (b & 0x3F);
        used++;
        lo = 0x80;
        hi = 0xBF;
    }
    *cp = v;
    return used;
}

template <size_t N>
bool in_ranges(const unsigned (&table)[N][2], uint32_t cp) {
    size_t lo = 0, hi = N;
    while (lo < hi) {
        const size_t mid = (lo + hi) / 2;
        if (cp < table[mid][0]) hi = mid;
        else if (cp > table[mid][1]) lo = mid + 1;
        else return true;
    }
    return false;
}

// ICU's \s: [\t\n\f\r\p{Z}]
bool is_space(uint32_t cp) {
    return cp == 9 || cp == 10 || cp == 12 || cp == 13 || cp == 0x20 || cp == 0xA0 || cp == 0x1680 || (cp >= 0x2000 && cp <= 0x200A) ||
           cp == 0x2028 || cp == 0x2029 || cp == 0x202F || cp == 0x205F || cp == 0x3000;
}
uint32_t fold_ascii(uint32_t cp) { return cp >= 'A' && cp <= 'Z' ? cp + 32 : cp; }

}  // namespace

std::vector<uint32_t> utf8_to_code_points(const std::string &s) {
    std::vector<uint32_t> out;
    out.reserve(s.size());
    for (size_t i = 0; i < s.size();) {
        uint32_t cp;
        bool ok;
        i += decode_one(s, i, &cp, &ok);
        out.push_back(cp);
    }
    return out;
}

void append_utf8(uint32_t cp, std::string *out) {
    if (cp >= 0x110000 || (cp >= 0xD800 && cp < 0xE000)) cp = 0xFFFD;
    if (cp < 0x80) out->push_back((char)cp);
    else if (cp < 0x800) { out->push_back((char)(0xC0 | (cp >> 6))); out->push_back((char)(0x80 | (cp & 0x3F))); }
    else if (cp < 0x10000) { out->push_back((char)(0xE0 | (cp >> 12))); out->push_back((char)(0x80 | ((cp >> 6) & 0x3F))); out->push_back((char)(0x80 | (cp & 0x3F))); }
    else { out->push_back((char)(0xF0 | (cp >> 18))); out->push_back((char)(0x80 | ((cp >> 12) & 0x3F))); out->push_back((char)(0x80 | ((cp >> 6) & 0x3F))); out->push_back((char)(0x80 | (cp & 0x3F))); }
}

std::string repair_utf8(const std::string &bytes) {
    std::string out;
    out.reserve(bytes.size());
    for (size_t i = 0; i < bytes.size();) {
        uint32_t cp;
        bool ok;
        const size_t used = decode_one(bytes, i, &cp, &ok);
        if (ok) out.append(bytes, i, used);
        else out += "\xEF\xBF\xBD";
        i += used;
    }
    return out;
}

bool unicode_is_letter(uint32_t cp) { return in_ranges(unicode_tables::kLetters, cp); }
bool unicode_is_number(uint32_t cp) { return in_ranges(unicode_tables::kNumbers, cp); }
bool unicode_is_extend(uint32_t cp) { return in_ranges(unicode_tables::kExtend, cp); }
bool unicode_is_spacing_mark(uint32_t cp) { return in_ranges(unicode_tables::kSpacingMarks, cp); }

// ---- pattern tree -----------------------------------------------------------------------------------

namespace {
struct ClassItem {
    enum Kind { Range, Letter, Number, Space, Digit } kind = Range;
    bool negate = false;   // \S, \D, \P{..}
    uint32_t lo = 0, hi = 0;
};
}  // namespace

struct Regex::Node {
    enum Type { Char, Any, Class, Group, Look, Bol, Eol } type = Char;
    uint32_t cp = 0;
    bool icase = false, negate = false;        // negate: [^...] or (?!...)
    std::vector<ClassItem> items;              // Class
    std::vector<std::vector<Node>> alts;       // Group, Look
    int min = 1, max = 1;                      // max < 0: unbounded
    bool lazy = false;
};

namespace {

using Node = Regex::Node;

struct Parser {
    const std::vector<uint32_t> &p;
    size_t i = 0;
    std::string err;
    bool fail(const std::string &m) { if (err.empty()) err = m + " at offset " + std::to_string(i); return false; }
    bool end() const { return i >= p.size(); }
    uint32_t peek(size_t k = 0) const { return i + k < p.size() ? p[i + k] : 0; }

    bool parse_hex(int digits_min, int digits_max, uint32_t stop, uint32_t *out) {
        uint32_t v = 0;
        int n = 0;
        while (!end() && n < digits_max) {
            const uint32_t c = peek();
            int d;
            if (c >= '0' && c <= '9') d = (int)(c - '0');
            else if (c >= 'a' && c <= 'f') d = (int)(c - 'a') + 10;
            else if (c >= 'A' && c <= 'F') d = (int)(c - 'A') + 10;
            else break;
            v = v * 16 + (uint32_t)d;
            n++;
            i++;
        }
        if (n < digits_min) return fail("bad hex escape");
        if (stop) { if (peek() != stop) return fail("bad hex escape"); i++; }
        *out = v;
        return true;
    }

    // After a backslash.  Either a class item (is_class) or a literal code point.
    bool parse_escape(ClassItem *item, bool *is_class, uint32_t *lit) {
        if (end()) return fail("trailing backslash");
        const uint32_t c = p[i++];
        *is_class = true;
        switch (c) {
        case 's': item->kind = ClassItem::Space; return true;
        case 'S': item->kind = ClassItem::Space; item->negate = true; return true;
        case 'd': item->kind = ClassItem::Digit; return true;
        case 'D': item->kind = ClassItem::Digit; item->negate = true; return true;
        case 'p': case 'P': {
            if (peek() != '{' || peek(2) != '}') return fail("unsupported property");
            const uint32_t name = peek(1);
            if (name == 'L') item->kind = ClassItem::Letter;
            else if (name == 'N') item->kind = ClassItem::Number;
            else return fail("unsupported property");
            item->negate = c == 'P';
            i += 3;
            return true;
        }
        default: break;
        }
        *is_class = false;
        switch (c) {
        case 'n': *lit = '\n'; return true;
        case 'r': *lit = '\r'; return true;
        case 't': *lit = '\t'; return true;
        case 'f': *lit = '\f'; return true;
        case 'v': *lit = 0x0B; return true;
        case 'u': return parse_hex(4, 4, 0, lit);
        case 'x':
            if (peek() == '{') { i++; return parse_hex(1, 6, '}', lit); }
            return parse_hex(2, 2, 0, lit);
        default: break;
        }
        if ((c >= 'a' && c <= 'z') || (c >= 'A' && c <= 'Z') || (c >= '0' && c <= '9')) return fail("unsupported escape");
        *lit = c;   // escaped punctuation
        return true;
    }

    bool parse_class(Node *n, bool icase) {
        n->type = Node::Class;
        n->icase = icase;
        if (peek() == '^') { n->negate = true; i++; }
        bool first = true;
        for (;;) {
            if (end()) return fail("unterminated class");
            uint32_t c = p[i];
            if (c == ']' && !first) { i++; return true; }
            first = false;
            if (c == '[') return fail("nested class");
            if (c == '&' && peek(1) == '&') return fail("class intersection");
            ClassItem item;
            i++;
            if (c == '\\') {
                bool is_class;
                uint32_t lit = 0;
                if (!parse_escape(&item, &is_class, &lit)) return false;
                if (is_class) { n->items.push_back(item); continue; }
                c = lit;
            }
            item.lo = item.hi = c;
            if (peek() == '-' && peek(1) != ']' && i + 1 < p.size()) {
                i++;
                uint32_t h = p[i++];
                if (h == '[') return fail("nested class");
                if (h == '\\') {
                    ClassItem tmp;
                    bool is_class;
                    if (!parse_escape(&tmp, &is_class, &h)) return false;
                    if (is_class) return fail("bad range");
                }
                if (h < c) return fail("bad range");
                item.hi = h;
            }
            n->items.push_back(item);
        }
    }

    bool parse_quantifier(Node *n) {
        const uint32_t c = peek();
        if (c == '*') { n->min = 0; n->max = -1; i++; }
        else if (c == '+') { n->min = 1; n->max = -1; i++; }
        else if (c == '?') { n->min = 0; n->max = 1; i++; }
        else if (c == '{') {
            i++;
            int lo = 0, hi = -2, digits = 0;
            while (peek() >= '0' && peek() <= '9') { lo = lo * 10 + (int)(p[i++] - '0'); if (++digits > 6) return fail("bad repeat"); }
            if (digits == 0) return fail("bad repeat");
            if (peek() == ',') {
                i++;
                if (peek() == '}') hi = -1;
                else {
                    hi = 0;
                    digits = 0;
                    while (peek() >= '0' && peek() <= '9') { hi = hi * 10 + (int)(p[i++] - '0'); if (++digits > 6) return fail("bad repeat"); }
                    if (digits == 0 || hi < lo) return fail("bad repeat");
                }
            } else hi = lo;
            if (peek() != '}') return fail("bad repeat");
            i++;
            n->min = lo;
            n->max = hi;
        } else return true;
        if (n->type == Node::Look || n->type == Node::Bol || n->type == Node::Eol) return fail("nothing to repeat");
        if (peek() == '?') { n->lazy = true; i++; }
        else if (peek() == '+') return fail("possessive quantifier");
        return true;
    }

    bool parse_alts(std::vector<std::vector<Node>> *alts, bool icase, int depth) {
        if (depth > 32) return fail("nesting too deep");
        alts->emplace_back();
        for (;;) {
            if (end()) return true;
            const uint32_t c = p[i];
            if (c == ')') return true;
            if (c == '|') { i++; alts->emplace_back(); continue; }
            Node n;
            n.icase = icase;
            i++;
            switch (c) {
            case '(': {
                bool group_icase = icase;
                n.type = Node::Group;
                if (peek() == '?') {
                    i++;
                    const uint32_t k = peek();
                    if (k == ':') i++;
                    else if (k == '=' || k == '!') { n.type = Node::Look; n.negate = k == '!'; i++; }
                    else if (k == 'i' && peek(1) == ':') { group_icase = true; i += 2; }
                    else if (k == 'i' && peek(1) == ')') { icase = true; i += 2; continue; }   // rest of this group
                    else return fail("unsupported group");
                }
                if (!parse_alts(&n.alts, group_icase, depth + 1)) return false;
                if (peek() != ')' || end()) return fail("missing )");
                i++;
                break;
            }
            case '[': if (!parse_class(&n, icase)) return false; break;
            case '.': n.type = Node::Any; break;
            case '^': n.type = Node::Bol; break;
            case '$': n.type = Node::Eol; break;
            case '*': case '+': case '?': case '{': return fail("nothing to repeat");
            case '\\': {
                ClassItem item;
                bool is_class;
                uint32_t lit = 0;
                if (!parse_escape(&item, &is_class, &lit)) return false;
                if (is_class) { n.type = Node::Class; n.items.push_back(item); }
                else { n.type = Node::Char; n.cp = lit; }
                break;
            }
            default: n.type = Node::Char; n.cp = c; break;
            }
            if (!parse_quantifier(&n)) return false;
            alts->back().push_back(std::move(n));
        }
    }
};

struct Matcher {
    const std::vector<uint32_t> &t;
    long steps = 0;
    static constexpr long kStepLimit = 20000000;   // gives up (no match) instead of running away
    using Cont = std::function<bool(size_t)>;

    static bool item_matches(const ClassItem &it, uint32_t c, bool icase) {
        bool m = false;
        switch (it.kind) {
        case ClassItem::Range:
            m = c >= it.lo && c <= it.hi;
            if (!m && icase) {
                const uint32_t f = fold_ascii(c), u = (c >= 'a' && c <= 'z') ? c - 32 : c;
                m = (f >= it.lo && f <= it.hi) || (u >= it.lo && u <= it.hi);
            }
            break;
        case ClassItem::Letter: m = unicode_is_letter(c); break;
        case ClassItem::Number: m = unicode_is_number(c); break;
        case ClassItem::Space: m = is_space(c); break;
        case ClassItem::Digit: m = in_ranges(unicode_tables::kDecimalDigits, c); break;
        }
        return m != it.negate;
    }

    bool single(const Node &n, size_t pos) const {   // one code point at pos against a one-character node
        if (pos >= t.size()) return false;
        const uint32_t c = t[pos];
        switch (n.type) {
        case Node::Char: return n.icase ? fold_ascii(c) == fold_ascii(n.cp) : c == n.cp;
        case Node::Any: return !(c >= 0x0A && c <= 0x0D) && c != 0x85 && c != 0x2028 && c != 0x2029;   // ICU's line terminators
        case Node::Class: {
            bool any = false;
            for (const ClassItem &it : n.items)
                if (item_matches(it, c, n.icase)) { any = true; break; }
            return any != n.negate;
        }
        default: return false;
        }
    }

    bool alts(const std::vector<std::vector<Node>> &a, size_t pos, const Cont &k) {
        for (const auto &seq : a)
            if (sequence(seq, 0, pos, k)) return true;
        return false;
    }

    bool sequence(const std::vector<Node> &seq, size_t idx, size_t pos, const Cont &k) {
        if (++steps > kStepLimit) return false;
        if (idx == seq.size()) return k(pos);
        const Node &n = seq[idx];
        const Cont next = [&](size_t q) { return sequence(seq, idx + 1, q, k); };
        switch (n.type) {
        case Node::Bol: return pos == 0 && next(pos);
        case Node::Eol: return pos == t.size() && next(pos);
        case Node::Look: {
            const bool found = alts(n.alts, pos, [](size_t) { return true; });
            return found != n.negate && next(pos);
        }
        case Node::Group: return repeat(n, 0, pos, next);
        default: return run(n, pos, next);
        }
    }

    // A repeated one-character node, without a stack frame per character: the longest run first
    // (the shortest first when lazy), then every shorter (longer) one.
    bool run(const Node &n, size_t pos, const Cont &k) {
        size_t longest = 0;
        while ((n.max < 0 || longest < (size_t)n.max) && single(n, pos + longest)) longest++;
        if (longest < (size_t)n.min) return false;
        if (n.lazy) {
            for (size_t len = (size_t)n.min; len <= longest; len++)
                if (k(pos + len)) return true;
            return false;
        }
        for (size_t len = longest + 1; len-- > (size_t)n.min;)
            if (k(pos + len)) return true;
        return false;
    }

    // `count` repetitions of n matched so far, the next one starting at pos
    bool repeat(const Node &n, int count, size_t pos, const Cont &k) {
        if (++steps > kStepLimit) return false;
        const bool may_stop = count >= n.min, may_go = n.max < 0 || count < n.max;
        const auto once = [&]() -> bool {
            if (!may_go) return false;
            if (n.type == Node::Group)
                return alts(n.alts, pos, [&](size_t q) { return (q != pos || count < n.min) && repeat(n, count + 1, q, k); });
            return single(n, pos) && repeat(n, count + 1, pos + 1, k);
        };
        if (n.lazy) return (may_stop && k(pos)) || once();
        return once() || (may_stop && k(pos));
    }
};

}  // namespace

Regex::Regex() = default;
Regex::~Regex() = default;
Regex::Regex(Regex &&) noexcept = default;
Regex &Regex::operator=(Regex &&) noexcept = default;

bool Regex::compile(const std::string &pattern_utf8, std::string *error) {
    const std::vector<uint32_t> p = utf8_to_code_points(pattern_utf8);
    Parser ps{p};
    auto root = std::make_unique<Node>();
    root->type = Node::Group;
    bool ok = ps.parse_alts(&root->alts, false, 0);
    if (ok && !ps.end()) ok = ps.fail("unbalanced )");
    if (!ok) {
        if (error) *error = ps.err;
        return false;
    }
    root_ = std::move(root);
    return true;
}

std::vector<std::pair<size_t, size_t>> Regex::matches(const std::vector<uint32_t> &text) const {
    std::vector<std::pair<size_t, size_t>> out;
    if (!root_) return out;
    Matcher m{text};
    size_t pos = 0;
    while (pos <= text.size()) {
        size_t end = 0;
        const bool hit = m.alts(root_->alts, pos, [&](size_t q) { end = q; return true; });
        if (m.steps > Matcher::kStepLimit) break;
        if (hit) {
            out.emplace_back(pos, end);
            pos = end > pos ? end : pos + 1;   // an empty match moves on by one
        } else pos++;
    }
    return out;
}

}  // namespace esp
