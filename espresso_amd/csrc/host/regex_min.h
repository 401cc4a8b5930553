// A small backtracking regular-expression matcher over Unicode code points: the subset of ICU syntax
// (NSRegularExpression) that BPE pre-tokenizer patterns use.
//   alternation |, groups (...), (?:...), (?i:...), (?i), look-ahead (?=...) (?!...)
//   quantifiers ? * + {m} {m,} {m,n}, each optionally lazy (a trailing ?)
//   classes [...] and [^...] with ranges and escapes, the dot, anchors ^ and $
//   escapes \s \S \d \D \w \W \p{L} \p{N} \P{L} \P{N} (also \p{Letter}-style long names are rejected),
//   \r \n \t \f \v \uXXXX \x{...} and escaped punctuation
// \s is ICU's [\t\n\f\r\p{Z}].  Leftmost match, alternatives in order, greedy quantifiers: the semantics
// of ICU's engine.  Anything else in a pattern makes compile() fail, as an invalid pattern would.
#pragma once

#include <cstdint>
#include <memory>
#include <string>
#include <utility>
#include <vector>

namespace esp {

// UTF-8 <-> code points.  Malformed input bytes decode to U+FFFD, one per maximal invalid subpart.
std::vector<uint32_t> utf8_to_code_points(const std::string &s);
void append_utf8(uint32_t cp, std::string *out);
// What String(decoding:as: UTF8.self) returns for arbitrary bytes: valid text kept, every maximal invalid
// subpart replaced by U+FFFD.
std::string repair_utf8(const std::string &bytes);

bool unicode_is_letter(uint32_t cp);         // general category L*
bool unicode_is_number(uint32_t cp);         // general category N*
bool unicode_is_extend(uint32_t cp);         // Mn | Me | U+200C | emoji modifiers
bool unicode_is_spacing_mark(uint32_t cp);   // Mc

class Regex {
  public:
    struct Node;
    Regex();
    ~Regex();
    Regex(Regex &&) noexcept;
    Regex &operator=(Regex &&) noexcept;
    // false (and *error set) when the pattern uses syntax outside the subset above
    bool compile(const std::string &pattern_utf8, std::string *error);
    // Non-overlapping matches from left to right as [begin, end) code-point offsets
    // (NSRegularExpression.matches(in:range:)); text between matches is skipped.
    std::vector<std::pair<size_t, size_t>> matches(const std::vector<uint32_t> &text) const;

  private:
    std::unique_ptr<Node> root_;
};

}  // namespace esp
