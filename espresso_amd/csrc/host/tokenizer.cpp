#include "tokenizer.h"

#include <cstdio>
#include <cstring>
#include <limits>

#include "json_min.h"

namespace esp {
namespace {

const char kMetaSpace[] = "\xE2\x96\x81";   // U+2581, the SentencePiece word-boundary mark

TokenizerStatus status(TokenizerError e, long detail = 0, long detail2 = 0, std::string text = {}) {
    TokenizerStatus s;
    s.error = e;
    s.detail = detail;
    s.detail2 = detail2;
    s.text = std::move(text);
    return s;
}

bool read_text(const std::string &path, std::string *out) {
    std::vector<uint8_t> raw;
    if (!readFile(path, &raw)) return false;
    out->assign(raw.begin(), raw.end());
    return true;
}

bool valid_utf8(const std::string &s) { return repair_utf8(s) == s; }

std::string replace_all(const std::string &s, const std::string &from, const std::string &to) {
    std::string out;
    size_t i = 0;
    for (;;) {
        const size_t j = s.find(from, i);
        if (j == std::string::npos) { out.append(s, i, std::string::npos); return out; }
        out.append(s, i, j - i);
        out += to;
        i = j + from.size();
    }
}

// ---- grapheme clusters ---------------------------------------------------------------------------------
enum class GB { Other, CR, LF, Control, Extend, ZWJ, SpacingMark, RI, L, V, T, LV, LVT, Pict };

GB gb_class(uint32_t c) {
    if (c == 0x0D) return GB::CR;
    if (c == 0x0A) return GB::LF;
    if (c == 0x200D) return GB::ZWJ;
    if (c < 0x20 || (c >= 0x7F && c <= 0x9F) || c == 0xAD || c == 0x200B || c == 0x200E || c == 0x200F || c == 0x2028 || c == 0x2029 ||
        (c >= 0x202A && c <= 0x202E) || (c >= 0x2060 && c <= 0x2064) || c == 0xFEFF || (c >= 0xFFF9 && c <= 0xFFFB))
        return GB::Control;
    if (unicode_is_extend(c) || (c >= 0xE0020 && c <= 0xE007F)) return GB::Extend;
    if (unicode_is_spacing_mark(c)) return GB::SpacingMark;
    if (c >= 0x1F1E6 && c <= 0x1F1FF) return GB::RI;
    if ((c >= 0x1100 && c <= 0x115F) || (c >= 0xA960 && c <= 0xA97C)) return GB::L;
    if ((c >= 0x1160 && c <= 0x11A7) || (c >= 0xD7B0 && c <= 0xD7C6)) return GB::V;
    if ((c >= 0x11A8 && c <= 0x11FF) || (c >= 0xD7CB && c <= 0xD7FB)) return GB::T;
    if (c >= 0xAC00 && c <= 0xD7A3) return (c - 0xAC00) % 28 == 0 ? GB::LV : GB::LVT;
    if (c == 0xA9 || c == 0xAE || c == 0x203C || c == 0x2049 || c == 0x2122 || c == 0x2139 || (c >= 0x2194 && c <= 0x21AA) ||
        (c >= 0x231A && c <= 0x23FF) || c == 0x24C2 || (c >= 0x25AA && c <= 0x25FE) || (c >= 0x2600 && c <= 0x27BF) ||
        c == 0x2934 || c == 0x2935 || (c >= 0x2B05 && c <= 0x2B55) || c == 0x3030 || c == 0x303D || c == 0x3297 || c == 0x3299 ||
        (c >= 0x1F000 && c <= 0x1FAFF))
        return GB::Pict;
    return GB::Other;
}

}  // namespace

std::vector<std::pair<size_t, size_t>> grapheme_clusters(const std::vector<uint32_t> &cps) {
    std::vector<std::pair<size_t, size_t>> out;
    if (cps.empty()) return out;
    size_t start = 0;
    GB prev = gb_class(cps[0]);
    int ri_run = prev == GB::RI ? 1 : 0;
    bool pict = prev == GB::Pict;       // cluster so far is ExtPict Extend*
    bool pict_zwj = false;              // ... followed by ZWJ
    for (size_t i = 1; i < cps.size(); i++) {
        const GB cur = gb_class(cps[i]);
        bool join;
        if (prev == GB::CR && cur == GB::LF) join = true;                                                     // GB3
        else if (prev == GB::CR || prev == GB::LF || prev == GB::Control) join = false;                      // GB4
        else if (cur == GB::CR || cur == GB::LF || cur == GB::Control) join = false;                         // GB5
        else if (prev == GB::L && (cur == GB::L || cur == GB::V || cur == GB::LV || cur == GB::LVT)) join = true;   // GB6
        else if ((prev == GB::LV || prev == GB::V) && (cur == GB::V || cur == GB::T)) join = true;           // GB7
        else if ((prev == GB::LVT || prev == GB::T) && cur == GB::T) join = true;                            // GB8
        else if (cur == GB::Extend || cur == GB::ZWJ || cur == GB::SpacingMark) join = true;                 // GB9, GB9a
        else if (pict_zwj && cur == GB::Pict) join = true;                                                   // GB11
        else if (prev == GB::RI && cur == GB::RI && ri_run % 2 == 1) join = true;                            // GB12, GB13
        else join = false;
        if (!join) {
            out.emplace_back(start, i);
            start = i;
            pict = cur == GB::Pict;
            pict_zwj = false;
            ri_run = cur == GB::RI ? 1 : 0;
        } else {
            if (cur == GB::Pict) { pict = true; pict_zwj = false; }
            else if (cur == GB::ZWJ) pict_zwj = pict;
            else if (cur == GB::Extend) pict_zwj = false;   // pict stays as it is
            else { pict = false; pict_zwj = false; }
            ri_run = cur == GB::RI ? ri_run + 1 : 0;
        }
        prev = cur;
    }
    out.emplace_back(start, cps.size());
    return out;
}

// ---- SentencePiece ---------------------------------------------------------------------------------------

TokenizerStatus SentencePieceTokenizer::load(const std::string &model_path, std::unique_ptr<SentencePieceTokenizer> *out) {
    std::string data;
    if (!read_text(model_path, &data)) return status(TokenizerError::UnreadableFile, 0, 0, model_path);
    return parse(data, out);
}

TokenizerStatus SentencePieceTokenizer::parse(const std::string &data, std::unique_ptr<SentencePieceTokenizer> *out) {
    if (data.size() < 4) return status(TokenizerError::SPTruncatedModel);
    size_t cursor = 0;
    const auto read_u32 = [&]() {
        uint32_t v = 0;
        for (int k = 0; k < 4; k++) v |= (uint32_t)(unsigned char)data[cursor + k] << (8 * k);
        cursor += 4;
        return v;
    };
    auto tok = std::unique_ptr<SentencePieceTokenizer>(new SentencePieceTokenizer());
    tok->max_token_length_ = (int32_t)read_u32();
    if (tok->max_token_length_ <= 0) return status(TokenizerError::SPInvalidMaxTokenLength, tok->max_token_length_);
    long index = 0;
    while (cursor < data.size()) {
        if (cursor + 8 > data.size()) return status(TokenizerError::SPTruncatedEntry, index);
        const uint32_t bits = read_u32();
        float score;
        std::memcpy(&score, &bits, 4);
        const int32_t length = (int32_t)read_u32();
        if (length < 0 || cursor + (size_t)length > data.size()) return status(TokenizerError::SPTruncatedEntry, index);
        std::string piece = data.substr(cursor, (size_t)length);
        cursor += (size_t)length;
        if (!valid_utf8(piece)) return status(TokenizerError::SPInvalidUTF8Entry, index);
        tok->piece_to_id_[piece] = (int)tok->pieces_.size();   // a repeated piece keeps its last id
        tok->pieces_.push_back(std::move(piece));
        tok->scores_.push_back(score);
        index++;
    }
    if (tok->pieces_.empty()) return status(TokenizerError::SPEmptyVocabulary);
    *out = std::move(tok);
    return {};
}

std::vector<int> SentencePieceTokenizer::encode(const std::string &text_utf8) const {
    const std::string normalized = kMetaSpace + replace_all(text_utf8, " ", kMetaSpace);
    const std::vector<uint32_t> cps = utf8_to_code_points(normalized);
    std::vector<int> tokens;
    for (const auto &cl : grapheme_clusters(cps)) {
        std::string piece;
        for (size_t i = cl.first; i < cl.second; i++) append_utf8(cps[i], &piece);
        const auto hit = piece_to_id_.find(piece);
        if (hit != piece_to_id_.end()) { tokens.push_back(hit->second); continue; }
        for (unsigned char byte : piece) {
            char fallback[8];
            std::snprintf(fallback, sizeof fallback, "<0x%02X>", byte);
            const auto fb = piece_to_id_.find(fallback);
            if (fb != piece_to_id_.end()) tokens.push_back(fb->second);
        }
    }
    // merge the adjacent pair whose concatenation has the highest score, leftmost on ties, until none is a piece
    while (tokens.size() >= 2) {
        float best_score = -std::numeric_limits<float>::max();
        long best_index = -1;
        int best_id = -1;
        for (size_t i = 0; i + 1 < tokens.size(); i++) {
            const std::string merged = pieces_[tokens[i]] + pieces_[tokens[i + 1]];
            if ((long)merged.size() > max_token_length_) continue;
            const auto hit = piece_to_id_.find(merged);
            if (hit == piece_to_id_.end()) continue;
            const float score = scores_[hit->second];
            if (score > best_score) { best_score = score; best_index = (long)i; best_id = hit->second; }
        }
        if (best_index < 0) break;
        tokens[(size_t)best_index] = best_id;
        tokens.erase(tokens.begin() + best_index + 1);
    }
    return tokens;
}

namespace {
// "<0xNN>" -> NN, as UInt8(_, radix: 16) reads the digits between "<0x" and ">"
bool byte_token(const std::string &piece, uint8_t *out) {
    if (piece.size() < 4 || piece.compare(0, 3, "<0x") != 0 || piece.back() != '>') return false;
    size_t i = 3;
    const size_t end = piece.size() - 1;
    if (i < end && piece[i] == '+') i++;
    if (i >= end) return false;
    unsigned v = 0;
    for (; i < end; i++) {
        const char c = piece[i];
        unsigned d;
        if (c >= '0' && c <= '9') d = (unsigned)(c - '0');
        else if (c >= 'a' && c <= 'f') d = (unsigned)(c - 'a') + 10;
        else if (c >= 'A' && c <= 'F') d = (unsigned)(c - 'A') + 10;
        else return false;
        v = v * 16 + d;
        if (v > 255) return false;
    }
    *out = (uint8_t)v;
    return true;
}
}  // namespace

std::string SentencePieceTokenizer::decode(const std::vector<int> &tokens) const {
    std::string bytes, text;
    for (int token : tokens) {
        if (token < 0 || (size_t)token >= pieces_.size()) continue;
        const std::string &piece = pieces_[(size_t)token];
        uint8_t b;
        if (byte_token(piece, &b)) { bytes.push_back((char)b); continue; }
        if (!bytes.empty()) { text += repair_utf8(bytes); bytes.clear(); }
        text += piece;
    }
    if (!bytes.empty()) text += repair_utf8(bytes);
    std::string restored = replace_all(text, kMetaSpace, " ");
    if (!restored.empty() && restored[0] == ' ') restored.erase(0, 1);
    return restored;
}

// ---- byte-level BPE ----------------------------------------------------------------------------------------

const char *GPT2BPETokenizer::defaultPreTokenizerPattern() {
    return "'s|'t|'re|'ve|'m|'ll|'d| ?\\p{L}+| ?\\p{N}+| ?[^\\s\\p{L}\\p{N}]+|\\s+";
}

namespace {

// parseVocabulary: every value a number (a JSON boolean is one to Foundation's NSNumber as well)
TokenizerStatus parse_vocabulary(const JsonNode &raw, std::map<std::string, long> *encoder) {
    if (raw.members.empty()) return status(TokenizerError::BPEEmptyVocabulary);
    for (const auto &m : raw.members) {
        if (m.second.is(JsonNode::Number)) (*encoder)[m.first] = (long)m.second.number;
        else if (m.second.is(JsonNode::Bool)) (*encoder)[m.first] = m.second.boolean ? 1 : 0;
        else return status(TokenizerError::BPEMalformedVocabulary);
    }
    return {};
}

bool all_objects(const JsonNode &array) {
    for (const JsonNode &n : array.items)
        if (!n.is(JsonNode::Object)) return false;
    return true;
}

std::vector<int> numeric_ids(const JsonNode &array) {
    std::vector<int> ids;
    for (const JsonNode &n : array.items)
        if (n.is(JsonNode::Number)) ids.push_back((int)n.number);
        else if (n.is(JsonNode::Bool)) ids.push_back(n.boolean ? 1 : 0);
    return ids;
}

bool find_regex_pattern(const JsonNode &pre, std::string *pattern) {
    const JsonNode *p = pre.find("pattern");
    if (p && p->is(JsonNode::Object)) {
        const JsonNode *r = p->find("Regex");
        if (r && r->is(JsonNode::String)) { *pattern = r->text; return true; }
    }
    const JsonNode *list = pre.find("pretokenizers");
    if (list && list->is(JsonNode::Array) && all_objects(*list))
        for (const JsonNode &entry : list->items)
            if (find_regex_pattern(entry, pattern)) return true;
    return false;
}

// prefixTokenIDs(in:): false = nil
bool prefix_ids_in(const JsonNode &processor, std::vector<int> *prefix) {
    const JsonNode *list = processor.find("processors");
    if (list && list->is(JsonNode::Array) && all_objects(*list))
        for (const JsonNode &entry : list->items)
            if (prefix_ids_in(entry, prefix)) return true;
    const JsonNode *special = processor.find("special_tokens");
    if (special && special->is(JsonNode::Object)) {
        const JsonNode *bos = special->find("<|begin_of_text|>");
        const JsonNode *ids = bos && bos->is(JsonNode::Object) ? bos->find("ids") : nullptr;
        if (ids && ids->is(JsonNode::Array)) {
            std::vector<int> v = numeric_ids(*ids);
            if (!v.empty()) { *prefix = std::move(v); return true; }
        }
    }
    const JsonNode *single = processor.find("single");
    if (!single || !single->is(JsonNode::Array) || !all_objects(*single)) return false;
    prefix->clear();
    for (const JsonNode &item : single->items) {
        const JsonNode *st = item.find("SpecialToken");
        const JsonNode *ids = st && st->is(JsonNode::Object) ? st->find("ids") : nullptr;
        if (ids && ids->is(JsonNode::Array)) {
            for (int id : numeric_ids(*ids)) prefix->push_back(id);
            continue;
        }
        if (item.find("Sequence")) break;
    }
    return true;
}

std::vector<std::string> split_omitting_empty(const std::string &s, char sep) {
    std::vector<std::string> out;
    size_t i = 0;
    while (i <= s.size()) {
        size_t j = s.find(sep, i);
        if (j == std::string::npos) j = s.size();
        if (j > i) out.push_back(s.substr(i, j - i));
        i = j + 1;
    }
    return out;
}

}  // namespace

TokenizerStatus GPT2BPETokenizer::load(const std::string &vocab_path, const std::string &merges_path, std::unique_ptr<GPT2BPETokenizer> *out) {
    std::string vocab_text, merges_text;
    if (!read_text(vocab_path, &vocab_text)) return status(TokenizerError::UnreadableFile, 0, 0, vocab_path);
    JsonNode root;
    std::string err;
    if (!json_parse(vocab_text, &root, &err) || !root.is(JsonNode::Object)) return status(TokenizerError::BPEMalformedVocabulary);
    if (!read_text(merges_path, &merges_text)) return status(TokenizerError::UnreadableFile, 0, 0, merges_path);
    std::map<std::string, long> encoder;
    TokenizerStatus st = parse_vocabulary(root, &encoder);
    if (!st.ok()) return st;
    return make(std::move(encoder), split_omitting_empty(merges_text, '\n'), defaultPreTokenizerPattern(), {}, {}, out);
}

TokenizerStatus GPT2BPETokenizer::loadTokenizerJSON(const std::string &path, std::unique_ptr<GPT2BPETokenizer> *out) {
    std::string text;
    if (!read_text(path, &text)) return status(TokenizerError::UnreadableFile, 0, 0, path);
    JsonNode root;
    std::string err;
    if (!json_parse(text, &root, &err) || !root.is(JsonNode::Object)) return status(TokenizerError::BPEMalformedTokenizerJSON);
    const JsonNode *model = root.find("model");
    if (!model || !model->is(JsonNode::Object)) return status(TokenizerError::BPEMalformedTokenizerJSON);
    const JsonNode *type = model->find("type");
    const std::string model_type = type && type->is(JsonNode::String) ? type->text : "unknown";
    if (model_type != "BPE") return status(TokenizerError::BPEUnsupportedTokenizerModel, 0, 0, model_type);
    const JsonNode *vocab = model->find("vocab");
    if (!vocab || !vocab->is(JsonNode::Object)) return status(TokenizerError::BPEMalformedTokenizerJSON);
    std::map<std::string, long> encoder;
    TokenizerStatus st = parse_vocabulary(*vocab, &encoder);
    if (!st.ok()) return st;

    // mergeAddedTokens: content -> id, special ones are left out of decoded text
    std::set<int> skipped;
    const JsonNode *added = root.find("added_tokens");
    if (added && added->is(JsonNode::Array) && all_objects(*added)) {
        for (const JsonNode &t : added->items) {
            const JsonNode *id = t.find("id"), *content = t.find("content"), *special = t.find("special");
            if (!id || !(id->is(JsonNode::Number) || id->is(JsonNode::Bool)) || !content || !content->is(JsonNode::String)) continue;
            const long v = id->is(JsonNode::Number) ? (long)id->number : (id->boolean ? 1 : 0);
            encoder[content->text] = v;
            if (special && special->is(JsonNode::Bool) && special->boolean) skipped.insert((int)v);
        }
    }

    // merges: ["a b", ...] or [["a", "b"], ...]
    const JsonNode *raw_merges = model->find("merges");
    if (!raw_merges || !raw_merges->is(JsonNode::Array)) return status(TokenizerError::BPEMalformedTokenizerJSON);
    std::vector<std::string> merges;
    bool all_strings = true, all_string_arrays = true;
    for (const JsonNode &m : raw_merges->items) {
        if (!m.is(JsonNode::String)) all_strings = false;
        if (!m.is(JsonNode::Array)) all_string_arrays = false;
        else
            for (const JsonNode &s : m.items)
                if (!s.is(JsonNode::String)) all_string_arrays = false;
    }
    if (all_strings) {
        for (const JsonNode &m : raw_merges->items) merges.push_back(m.text);
    } else if (all_string_arrays) {
        for (const JsonNode &m : raw_merges->items)
            if (m.items.size() == 2) merges.push_back(m.items[0].text + " " + m.items[1].text);
    } else return status(TokenizerError::BPEMalformedTokenizerJSON);

    std::string pattern = defaultPreTokenizerPattern();
    const JsonNode *pre = root.find("pre_tokenizer");
    if (pre && pre->is(JsonNode::Object)) {
        std::string found;
        if (find_regex_pattern(*pre, &found)) pattern = found;
    }

    std::vector<int> prefix;
    const JsonNode *post = root.find("post_processor");
    if (!(post && post->is(JsonNode::Object) && prefix_ids_in(*post, &prefix) && !prefix.empty())) {
        prefix.clear();
        const auto bos = encoder.find("<|begin_of_text|>");
        if (bos != encoder.end()) prefix.push_back((int)bos->second);
    }
    return make(std::move(encoder), merges, pattern, std::move(prefix), std::move(skipped), out);
}

TokenizerStatus GPT2BPETokenizer::make(std::map<std::string, long> encoder, const std::vector<std::string> &merges, const std::string &pattern,
                                       std::vector<int> prefix, std::set<int> skipped, std::unique_ptr<GPT2BPETokenizer> *out) {
    if (encoder.empty()) return status(TokenizerError::BPEEmptyVocabulary);
    long max_id = -1;
    for (const auto &e : encoder) max_id = e.second > max_id ? e.second : max_id;
    if (max_id < 0) return status(TokenizerError::BPEEmptyVocabulary);
    if (max_id + 1 != (long)encoder.size()) return status(TokenizerError::BPENonContiguousTokenIDs, (long)encoder.size(), max_id);

    auto tok = std::unique_ptr<GPT2BPETokenizer>(new GPT2BPETokenizer());
    tok->decoder_.assign((size_t)max_id + 1, std::string());
    for (const auto &e : encoder) {
        tok->encoder_[e.first] = (int)e.second;
        if (e.second >= 0) tok->decoder_[(size_t)e.second] = e.first;
    }
    tok->prefix_ = std::move(prefix);
    tok->skipped_ = std::move(skipped);

    int rank = 0;
    for (const std::string &line : merges) {
        if (line.empty() || line[0] == '#') continue;
        const std::vector<std::string> parts = split_omitting_empty(line, ' ');
        if (parts.size() != 2) continue;
        tok->ranks_[parts[0] + std::string(1, '\0') + parts[1]] = rank++;
    }

    // the byte <-> printable code point table of GPT-2: printable Latin-1 bytes stand for themselves, the
    // rest take U+0100 upwards in byte order
    bool direct[256] = {};
    for (int b = 33; b <= 126; b++) direct[b] = true;
    for (int b = 161; b <= 172; b++) direct[b] = true;
    for (int b = 174; b <= 255; b++) direct[b] = true;
    uint32_t next = 256;
    for (int b = 0; b < 256; b++) {
        tok->byte_to_unicode_[b] = direct[b] ? (uint32_t)b : next++;
        tok->unicode_to_byte_[tok->byte_to_unicode_[b]] = (uint8_t)b;
    }

    std::string err;
    if (!tok->pre_tokenizer_.compile(pattern, &err)) return status(TokenizerError::BPEInvalidPreTokenizerPattern, 0, 0, pattern);
    *out = std::move(tok);
    return {};
}

std::vector<std::string> GPT2BPETokenizer::bpe(const std::string &token) const {
    std::vector<std::string> word;
    for (uint32_t cp : utf8_to_code_points(token)) {
        word.emplace_back();
        append_utf8(cp, &word.back());
    }
    while (word.size() > 1) {
        int best_rank = std::numeric_limits<int>::max();
        size_t best = word.size();
        for (size_t i = 0; i + 1 < word.size(); i++) {
            const auto hit = ranks_.find(word[i] + std::string(1, '\0') + word[i + 1]);
            if (hit != ranks_.end() && hit->second < best_rank) { best_rank = hit->second; best = i; }
        }
        if (best == word.size()) break;
        const std::string left = word[best], right = word[best + 1];
        std::vector<std::string> merged;
        for (size_t i = 0; i < word.size();) {
            if (i + 1 < word.size() && word[i] == left && word[i + 1] == right) { merged.push_back(left + right); i += 2; }
            else { merged.push_back(word[i]); i += 1; }
        }
        word = std::move(merged);
    }
    return word;
}

std::vector<int> GPT2BPETokenizer::encode(const std::string &text_utf8) const {
    const std::vector<uint32_t> cps = utf8_to_code_points(text_utf8);
    std::vector<int> tokens = prefix_;
    for (const auto &m : pre_tokenizer_.matches(cps)) {
        std::string chunk, mapped;
        for (size_t i = m.first; i < m.second; i++) append_utf8(cps[i], &chunk);
        for (unsigned char b : chunk) append_utf8(byte_to_unicode_[b], &mapped);
        for (const std::string &piece : bpe(mapped)) {
            const auto hit = encoder_.find(piece);
            if (hit != encoder_.end()) tokens.push_back(hit->second);
        }
    }
    return tokens;
}

std::string GPT2BPETokenizer::decode(const std::vector<int> &tokens) const {
    std::string bytes;
    for (int token : tokens) {
        if (token < 0 || (size_t)token >= decoder_.size() || skipped_.count(token)) continue;
        for (uint32_t cp : utf8_to_code_points(decoder_[(size_t)token])) {
            const auto hit = unicode_to_byte_.find(cp);
            if (hit != unicode_to_byte_.end()) bytes.push_back((char)hit->second);
            else append_utf8(cp, &bytes);
        }
    }
    return repair_utf8(bytes);
}

// ---- selection -------------------------------------------------------------------------------------------

TokenizerStatus loadTokenizer(const MultiModelConfig &config, const std::string &dir, std::unique_ptr<Tokenizer> *out) {
    const std::string vocab = joinPath(dir, "vocab.json"), merges = joinPath(dir, "merges.txt");
    const auto load_bpe = [&](std::unique_ptr<Tokenizer> *o) {
        std::unique_ptr<GPT2BPETokenizer> t;
        TokenizerStatus st = GPT2BPETokenizer::load(vocab, merges, &t);
        if (st.ok()) *o = std::move(t);
        return st;
    };
    if (config.architecture == MultiModelConfig::Architecture::gpt2) {
        if (!fileExists(vocab)) return status(TokenizerError::MissingPath, 0, 0, vocab);
        if (!fileExists(merges)) return status(TokenizerError::MissingPath, 0, 0, merges);
        return load_bpe(out);
    }
    for (const char *candidate : {"tokenizer.model", "tokenizer.bin"}) {
        const std::string path = joinPath(dir, candidate);
        if (!fileExists(path)) continue;
        std::unique_ptr<SentencePieceTokenizer> t;
        TokenizerStatus st = SentencePieceTokenizer::load(path, &t);
        if (st.ok()) *out = std::move(t);
        return st;
    }
    const std::string tokenizer_json = joinPath(dir, "tokenizer.json");
    if (fileExists(tokenizer_json)) {
        std::unique_ptr<GPT2BPETokenizer> t;
        TokenizerStatus st = GPT2BPETokenizer::loadTokenizerJSON(tokenizer_json, &t);
        if (st.ok()) *out = std::move(t);
        return st;
    }
    if (fileExists(vocab) && fileExists(merges)) return load_bpe(out);
    return status(TokenizerError::MissingPath, 0, 0,
                  "No tokenizer found in " + dir + " - tried tokenizer.model, tokenizer.bin, tokenizer.json, vocab.json+merges.txt");
}

}  // namespace esp
