// Text <-> token ids for generate(prompt:): the reference's two tokenizers and its selection order.
//   Tokenizer protocol              Sources/ModelSupport/Tokenizer.swift:1-5
//   SentencePieceTokenizer          Sources/ModelSupport/SentencePieceTokenizer.swift:11-146
//   GPT2BPETokenizer                Sources/ModelSupport/GPT2BPETokenizer.swift:12-381
//   loadTokenizer (selection order) Sources/RealModelInference/RealModelInferenceEngine.swift:7558-7613
#pragma once

#include <cstdint>
#include <map>
#include <memory>
#include <set>
#include <string>
#include <unordered_map>
#include <vector>

#include "model_support.h"
#include "regex_min.h"

namespace esp {

// Error cases of SentencePieceTokenizerError and GPT2BPETokenizerError, flattened.
enum class TokenizerError : int {
    None = 0,
    UnreadableFile = 1,
    SPTruncatedModel = 10,
    SPInvalidMaxTokenLength = 11,   // detail = the value
    SPTruncatedEntry = 12,          // detail = entry index
    SPInvalidUTF8Entry = 13,        // detail = entry index
    SPEmptyVocabulary = 14,
    BPEMalformedVocabulary = 20,
    BPEEmptyVocabulary = 21,
    BPENonContiguousTokenIDs = 22,   // detail = expectedCount, detail2 = actualMaxTokenID
    BPEMalformedTokenizerJSON = 23,
    BPEUnsupportedTokenizerModel = 24,      // text = the model type
    BPEInvalidPreTokenizerPattern = 25,     // text = the pattern
    MissingPath = 30,                       // text = what was looked for
};

struct TokenizerStatus {
    TokenizerError error = TokenizerError::None;
    long detail = 0, detail2 = 0;
    std::string text;
    bool ok() const { return error == TokenizerError::None; }
};

class Tokenizer {
  public:
    virtual ~Tokenizer() = default;
    virtual std::vector<int> encode(const std::string &text_utf8) const = 0;
    virtual std::string decode(const std::vector<int> &tokens) const = 0;
    virtual int vocabSize() const = 0;
    virtual const char *kind() const = 0;   // "sentencePiece" or "gpt2", the cases of LoadedTokenizer
};

// The flat binary vocabulary (int32 maxTokenLength, then per piece float32 score, int32 byte length,
// UTF-8 bytes; all little-endian) with greedy best-score pair merging and <0xNN> byte fallback.
class SentencePieceTokenizer : public Tokenizer {
  public:
    static TokenizerStatus load(const std::string &model_path, std::unique_ptr<SentencePieceTokenizer> *out);
    static TokenizerStatus parse(const std::string &data, std::unique_ptr<SentencePieceTokenizer> *out);
    std::vector<int> encode(const std::string &text_utf8) const override;
    std::string decode(const std::vector<int> &tokens) const override;
    int vocabSize() const override { return (int)pieces_.size(); }
    const char *kind() const override { return "sentencePiece"; }

  private:
    std::vector<std::string> pieces_;
    std::vector<float> scores_;
    std::unordered_map<std::string, int> piece_to_id_;
    int max_token_length_ = 0;
};

// Byte-level BPE from vocab.json + merges.txt, or from a tokenizer.json (model.type "BPE", added_tokens,
// pre_tokenizer pattern, post_processor prefix ids).
class GPT2BPETokenizer : public Tokenizer {
  public:
    static TokenizerStatus load(const std::string &vocab_path, const std::string &merges_path, std::unique_ptr<GPT2BPETokenizer> *out);
    static TokenizerStatus loadTokenizerJSON(const std::string &tokenizer_json_path, std::unique_ptr<GPT2BPETokenizer> *out);
    std::vector<int> encode(const std::string &text_utf8) const override;
    std::string decode(const std::vector<int> &tokens) const override;
    int vocabSize() const override { return (int)decoder_.size(); }
    const char *kind() const override { return "gpt2"; }
    static const char *defaultPreTokenizerPattern();

  private:
    static TokenizerStatus make(std::map<std::string, long> encoder, const std::vector<std::string> &merges, const std::string &pattern,
                                std::vector<int> prefix, std::set<int> skipped, std::unique_ptr<GPT2BPETokenizer> *out);
    std::vector<std::string> bpe(const std::string &token) const;
    std::unordered_map<std::string, int> encoder_;
    std::vector<std::string> decoder_;
    std::unordered_map<std::string, int> ranks_;   // key: left + '\0' + right
    uint32_t byte_to_unicode_[256];
    std::unordered_map<uint32_t, uint8_t> unicode_to_byte_;
    Regex pre_tokenizer_;
    std::vector<int> prefix_;
    std::set<int> skipped_;
};

// loadTokenizer(config:tokenizerDirURL:): gpt2 -> vocab.json + merges.txt; llama -> tokenizer.model, tokenizer.bin
// (SentencePiece), tokenizer.json, vocab.json + merges.txt, in that order; none -> MissingPath.
TokenizerStatus loadTokenizer(const MultiModelConfig &config, const std::string &tokenizer_dir, std::unique_ptr<Tokenizer> *out);

// Extended grapheme clusters of `cps` as [begin, end) ranges: what iterating a Swift String yields.
// Rules GB3-GB13 of UAX #29 with Extend = Mn | Me | U+200C | emoji modifiers, SpacingMark = Mc, and
// "extended pictographic" taken as U+00A9, U+00AE, U+203C-U+3299 symbols blocks and U+1F000-U+1FAFF.
std::vector<std::pair<size_t, size_t>> grapheme_clusters(const std::vector<uint32_t> &cps);

}  // namespace esp
