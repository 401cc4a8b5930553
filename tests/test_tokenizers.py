"""Tokenizers (host code, no GPU): the reference's own test vectors (Tests/ModelSupportTests/TokenizerTests.swift),
then independent checks of the parts those leave open: the pre-tokenizer against the `regex` module, byte-level
BPE against the Hugging Face `tokenizers` library (the reference's own yardstick for this class,
TokenizerTests.swift:37-47), SentencePiece merging against a plain restatement of
SentencePieceTokenizer.swift:68-112."""
import json
import random
import struct

import pytest

from espresso_amd import tokenizer as T
from espresso_amd.llama import MultiModelConfig

LLAMA3_PATTERN = (r"(?i:'s|'t|'re|'ve|'m|'ll|'d)|[^\r\n\p{L}\p{N}]?\p{L}+|\p{N}{1,3}| ?[^\s\p{L}\p{N}]+[\r\n]*|\s*[\r\n]+|\s+(?!\S)|\s+")
GPT2_PATTERN = r"'s|'t|'re|'ve|'m|'ll|'d| ?\p{L}+| ?\p{N}+| ?[^\s\p{L}\p{N}]+|\s+"


def gpt2_byte_unicode_map():
    printable = list(range(33, 127)) + list(range(161, 173)) + list(range(174, 256))
    mapped = list(printable)
    extra = 0
    for value in range(256):
        if value not in printable:
            printable.append(value)
            mapped.append(256 + extra)
            extra += 1
    return {b: chr(m) for b, m in zip(printable, mapped)}


BYTE_MAP = gpt2_byte_unicode_map()
NEWLINE, SPACE = BYTE_MAP[10], BYTE_MAP[32]
FIXTURE_VOCAB = {"Hello": 0, ",": 1, f"{SPACE}world": 2, "!": 3, NEWLINE: 4}
FIXTURE_MERGES = ["H e", "He l", "Hel l", "Hell o", f"{SPACE} w", f"{SPACE}w o", f"{SPACE}wo r", f"{SPACE}wor l", f"{SPACE}worl d"]


# ---- the reference's fixtures (TokenizerTests.swift:152-279), rebuilt from the data listed there ----
def make_gpt2_fixture(tmp_path):
    vocab, merges = tmp_path / "vocab.json", tmp_path / "merges.txt"
    vocab.write_text(json.dumps(FIXTURE_VOCAB, sort_keys=True), encoding="utf-8")
    merges.write_text("\n".join(["#version: 0.2"] + FIXTURE_MERGES), encoding="utf-8")
    return str(vocab), str(merges)


def make_tokenizer_json_fixture(tmp_path):
    payload = {
        "added_tokens": [{"id": 5, "content": "<|begin_of_text|>", "special": True, "single_word": False, "lstrip": False,
                          "rstrip": False, "normalized": False}],
        "pre_tokenizer": {"type": "Sequence", "pretokenizers": [
            {"type": "Split", "pattern": {"Regex": GPT2_PATTERN}, "behavior": "Isolated", "invert": False}]},
        "post_processor": {"type": "Sequence", "processors": [{"type": "TemplateProcessing", "single": [
            {"SpecialToken": {"id": "<|begin_of_text|>", "ids": [5], "tokens": ["<|begin_of_text|>"]}},
            {"Sequence": {"id": "A", "type_id": 0}}]}]},
        "model": {"type": "BPE", "vocab": FIXTURE_VOCAB, "merges": FIXTURE_MERGES},
    }
    path = tmp_path / "tokenizer.json"
    path.write_text(json.dumps(payload, sort_keys=True), encoding="utf-8")
    return str(path)


SP_PIECES = [("▁", 0.0), ("H", 0.0), ("e", 0.0), ("l", 0.0), ("o", 0.0), (",", 0.0), ("w", 0.0), ("r", 0.0), ("d", 0.0), ("!", 0.0),
             ("▁H", 1.0), ("▁He", 2.0), ("▁Hel", 3.0), ("▁Hell", 4.0), ("▁Hello", 5.0), ("▁w", 1.0), ("▁wo", 2.0), ("▁wor", 3.0),
             ("▁worl", 4.0), ("▁world", 5.0), ("<0x0A>", 0.0)]


def sp_model_bytes(pieces, max_token_length=16):
    data = struct.pack("<i", max_token_length)
    for piece, score in pieces:
        raw = piece.encode("utf-8")
        data += struct.pack("<fi", score, len(raw)) + raw
    return data


def make_sp_fixture(tmp_path, pieces=SP_PIECES, name="tokenizer.model"):
    path = tmp_path / name
    path.write_bytes(sp_model_bytes(pieces))
    return str(path)


# ---- TokenizerTests.swift:5-19 ----
def test_gpt2_round_trips_hello_world_and_non_printable_bytes(tmp_path):
    tok = T.Tokenizer.gpt2(*make_gpt2_fixture(tmp_path))
    assert tok.kind == "gpt2" and tok.vocab_size == 5
    encoded = tok.encode("Hello, world!")
    assert encoded == [0, 1, 2, 3]
    assert tok.decode(encoded) == "Hello, world!"
    assert tok.encode("\n") == [4]
    assert tok.decode([4]) == "\n"


# ---- TokenizerTests.swift:21-35 ----
def test_tokenizer_json_round_trips_and_skips_special_tokens(tmp_path):
    tok = T.Tokenizer.tokenizer_json(make_tokenizer_json_fixture(tmp_path))
    assert tok.vocab_size == 6
    encoded = tok.encode("Hello, world!")
    assert encoded == [5, 0, 1, 2, 3]
    assert tok.decode(encoded) == "Hello, world!"
    assert tok.encode("\n") == [5, 4]
    assert tok.decode([5, 4]) == "\n"


def test_tokenizer_json_merges_as_pairs_and_bos_fallback(tmp_path):
    # merges as [["a","b"],...] (GPT2BPETokenizer.swift:308-313); without a post-processor the prefix is the id of
    # "<|begin_of_text|>" when the vocabulary has one (:338-343)
    payload = {"added_tokens": [{"id": 5, "content": "<|begin_of_text|>", "special": True}],
               "model": {"type": "BPE", "vocab": FIXTURE_VOCAB, "merges": [m.split(" ") for m in FIXTURE_MERGES]}}
    path = tmp_path / "tokenizer.json"
    path.write_text(json.dumps(payload), encoding="utf-8")
    tok = T.Tokenizer.tokenizer_json(str(path))
    assert tok.encode("Hello, world!") == [5, 0, 1, 2, 3]


# ---- TokenizerTests.swift:49-60 ----
def test_sentencepiece_round_trips_hello_world_and_byte_fallback(tmp_path):
    tok = T.Tokenizer.sentencepiece(make_sp_fixture(tmp_path))
    assert tok.kind == "sentencePiece" and tok.vocab_size == len(SP_PIECES)
    encoded = tok.encode("Hello, world!")
    # "▁Hello,▁world!": the 1.0 merges first (leftmost), then 2.0 ... 5.0 on each word
    assert encoded == [14, 5, 19, 9]
    assert tok.decode(encoded) == "Hello, world!"
    newline = tok.encode("\n")
    assert newline == [0, 20]          # "▁" then the byte piece <0x0A>
    assert tok.decode(newline) == "\n"


# ---- TokenizerTests.swift:62-149: the error cases ----
def test_gpt2_rejects_malformed_vocabulary(tmp_path):
    (tmp_path / "vocab.json").write_text('["not","a","map"]')
    (tmp_path / "merges.txt").write_text("#version: 0.2\n")
    with pytest.raises(T.TokenizerError) as e:
        T.Tokenizer.gpt2(str(tmp_path / "vocab.json"), str(tmp_path / "merges.txt"))
    assert e.value.case == "malformedVocabulary"


def test_gpt2_rejects_non_contiguous_vocabulary_ids(tmp_path):
    (tmp_path / "vocab.json").write_text(json.dumps({"a": 0, "b": 2}))
    (tmp_path / "merges.txt").write_text("#version: 0.2\n")
    with pytest.raises(T.TokenizerError) as e:
        T.Tokenizer.gpt2(str(tmp_path / "vocab.json"), str(tmp_path / "merges.txt"))
    assert (e.value.case, e.value.detail, e.value.detail2) == ("nonContiguousTokenIDs", 2, 2)


def test_tokenizer_json_rejects_unsupported_model_type(tmp_path):
    (tmp_path / "tokenizer.json").write_text(json.dumps({"model": {"type": "WordPiece", "vocab": {"a": 0}, "merges": []}}))
    with pytest.raises(T.TokenizerError) as e:
        T.Tokenizer.tokenizer_json(str(tmp_path / "tokenizer.json"))
    assert (e.value.case, e.value.text) == ("unsupportedTokenizerModel", "WordPiece")


def test_sentencepiece_rejects_truncated_model(tmp_path):
    (tmp_path / "tokenizer.model").write_bytes(bytes([1, 2]))
    with pytest.raises(T.TokenizerError) as e:
        T.Tokenizer.sentencepiece(str(tmp_path / "tokenizer.model"))
    assert e.value.case == "truncatedModel"


def test_sentencepiece_rejects_truncated_entry(tmp_path):
    (tmp_path / "tokenizer.model").write_bytes(struct.pack("<ifi", 8, 0.0, 4) + b"ab")
    with pytest.raises(T.TokenizerError) as e:
        T.Tokenizer.sentencepiece(str(tmp_path / "tokenizer.model"))
    assert (e.value.case, e.value.detail) == ("truncatedEntry", 0)


def test_other_load_errors(tmp_path):
    (tmp_path / "a.model").write_bytes(struct.pack("<i", 0))
    with pytest.raises(T.TokenizerError) as e:
        T.Tokenizer.sentencepiece(str(tmp_path / "a.model"))
    assert (e.value.case, e.value.detail) == ("invalidMaxTokenLength", 0)
    (tmp_path / "b.model").write_bytes(struct.pack("<i", 8))
    with pytest.raises(T.TokenizerError) as e:
        T.Tokenizer.sentencepiece(str(tmp_path / "b.model"))
    assert e.value.case == "emptyVocabulary"
    (tmp_path / "c.model").write_bytes(struct.pack("<ifi", 8, 0.0, 2) + b"\xff\xfe")
    with pytest.raises(T.TokenizerError) as e:
        T.Tokenizer.sentencepiece(str(tmp_path / "c.model"))
    assert (e.value.case, e.value.detail) == ("invalidUTF8Entry", 0)
    (tmp_path / "tokenizer.json").write_text(json.dumps({"model": {"type": "BPE", "vocab": {"a": 0}, "merges": []},
                                                         "pre_tokenizer": {"pattern": {"Regex": "(?<=a)b"}}}))
    with pytest.raises(T.TokenizerError) as e:
        T.Tokenizer.tokenizer_json(str(tmp_path / "tokenizer.json"))
    assert (e.value.case, e.value.text) == ("invalidPreTokenizerPattern", "(?<=a)b")
    (tmp_path / "t2.json").write_text(json.dumps({"model": {"type": "BPE", "vocab": {"a": 0}}}))
    with pytest.raises(T.TokenizerError) as e:
        T.Tokenizer.tokenizer_json(str(tmp_path / "t2.json"))
    assert e.value.case == "malformedTokenizerJSON"


# ---- loadTokenizer (RealModelInferenceEngine.swift:7558-7613): the order of candidates ----
def test_directory_selection_order(tmp_path):
    cfg = MultiModelConfig(n_layer=1, n_head=1, n_kv_head=1, d_model=8, head_dim=8, hidden_dim=16, vocab=32, max_seq=16)
    d = tmp_path / "tok"
    d.mkdir()
    with pytest.raises(T.TokenizerError) as e:
        T.Tokenizer.from_dir(cfg, str(d))
    assert e.value.case == "missingPath" and "tokenizer.model, tokenizer.bin, tokenizer.json, vocab.json+merges.txt" in e.value.text
    make_gpt2_fixture(d)
    assert T.Tokenizer.from_dir(cfg, str(d)).encode("\n") == [4]                 # vocab.json + merges.txt: the last resort
    make_tokenizer_json_fixture(d)
    assert T.Tokenizer.from_dir(cfg, str(d)).encode("\n") == [5, 4]              # tokenizer.json before them
    make_sp_fixture(d, name="tokenizer.bin")
    assert T.Tokenizer.from_dir(cfg, str(d)).kind == "sentencePiece"             # SentencePiece first
    make_sp_fixture(d, pieces=SP_PIECES[:10], name="tokenizer.model")
    assert T.Tokenizer.from_dir(cfg, str(d)).vocab_size == 10                    # tokenizer.model before tokenizer.bin
    # architecture gpt2 reads vocab.json + merges.txt only
    assert T.Tokenizer.from_dir(cfg, str(d), architecture="gpt2").kind == "gpt2"
    (d / "merges.txt").unlink()
    with pytest.raises(T.TokenizerError) as e:
        T.Tokenizer.from_dir(cfg, str(d), architecture="gpt2")
    assert e.value.case == "missingPath" and e.value.text.endswith("merges.txt")


# ---- pre-tokenizer against the `regex` module ----
ALPHABET = list("abcXYZ éßЖдя 中文字 ٣७9 012  \t\n\r\n'`!?.,;:-_()[]{}#@&*+=/\\|~^%$\"<>") + ["'s", "'T", "'re", "'ll", " ", "  ", "\n\n", "é",
                                                                                          " ", "　", "😀", "½", "Ⅷ"]


def random_text(rng, n):
    return "".join(rng.choice(ALPHABET) for _ in range(n))


@pytest.mark.parametrize("pattern", [GPT2_PATTERN, LLAMA3_PATTERN, r"\p{N}{2,}?|\P{L}|[a-c-]+|[^\S\n]*$", r"(?i)x[y-z]+|(?:ab|a)(?=c)|\d+|[^\r\n]"])
def test_pretokenizer_matches_regex_module(pattern):
    regex = pytest.importorskip("regex")
    # ICU's \s is [\t\n\f\r\p{Z}]; the alphabet holds no character on which the module's \s differs
    compiled = regex.compile(pattern)
    rng = random.Random(7)
    for trial in range(300):
        text = random_text(rng, rng.randint(0, 40))
        want = [m.group(0) for m in compiled.finditer(text)]
        got = T.pretokenize(text, pattern)
        assert [g for g in got if g != ""] == [w for w in want if w != ""], (pattern, text)


def test_pretokenizer_rejects_syntax_outside_the_subset():
    for bad in ["(?<=a)b", "a++", "[[:alpha:]]", r"\p{Greek}", "(", "a)", "*a", r"\w+", "a{2,1}"]:
        with pytest.raises(Exception):
            T.pretokenize("abc", bad)


# ---- byte-level BPE against Hugging Face tokenizers ----
def train_bpe(corpus_words, merges_wanted):
    """A plain BPE trainer over byte-mapped words: most frequent adjacent pair first, ties by order of appearance."""
    words = [[BYTE_MAP[b] for b in w.encode("utf-8")] for w in corpus_words]
    merges = []
    for _ in range(merges_wanted):
        counts = {}
        for w in words:
            for a, b in zip(w, w[1:]):
                counts[(a, b)] = counts.get((a, b), 0) + 1
        if not counts:
            break
        best = max(counts, key=lambda p: counts[p])
        if counts[best] < 2:
            break
        merges.append(best)
        for i, w in enumerate(words):
            out, j = [], 0
            while j < len(w):
                if j + 1 < len(w) and (w[j], w[j + 1]) == best:
                    out.append(w[j] + w[j + 1]); j += 2
                else:
                    out.append(w[j]); j += 1
            words[i] = out
    return merges


@pytest.mark.parametrize("pattern", [GPT2_PATTERN, LLAMA3_PATTERN])
def test_byte_level_bpe_matches_huggingface_tokenizers(tmp_path, pattern):
    hf = pytest.importorskip("tokenizers")
    rng = random.Random(11)
    corpus = [random_text(rng, rng.randint(1, 12)) for _ in range(400)] + ["hello world", "the quick brown fox", "中文字中文"] * 20
    merges = train_bpe(corpus, 150)
    vocab = {BYTE_MAP[b]: i for i, b in enumerate(range(256))}
    for a, b in merges:
        vocab.setdefault(a + b, len(vocab))
    bos = len(vocab)
    payload = {
        "version": "1.0", "truncation": None, "padding": None,
        "added_tokens": [{"id": bos, "content": "<|begin_of_text|>", "single_word": False, "lstrip": False, "rstrip": False,
                          "normalized": False, "special": True}],
        "normalizer": None,
        "pre_tokenizer": {"type": "Sequence", "pretokenizers": [
            {"type": "Split", "pattern": {"Regex": pattern}, "behavior": "Isolated", "invert": False},
            {"type": "ByteLevel", "add_prefix_space": False, "trim_offsets": True, "use_regex": False}]},
        "post_processor": {"type": "TemplateProcessing",
                           "single": [{"SpecialToken": {"id": "<|begin_of_text|>", "type_id": 0}}, {"Sequence": {"id": "A", "type_id": 0}}],
                           "pair": [{"Sequence": {"id": "A", "type_id": 0}}, {"Sequence": {"id": "B", "type_id": 1}}],
                           "special_tokens": {"<|begin_of_text|>": {"id": "<|begin_of_text|>", "ids": [bos], "tokens": ["<|begin_of_text|>"]}}},
        "decoder": {"type": "ByteLevel", "add_prefix_space": True, "trim_offsets": True, "use_regex": True},
        "model": {"type": "BPE", "dropout": None, "unk_token": None, "continuing_subword_prefix": None, "end_of_word_suffix": None,
                  "fuse_unk": False, "byte_fallback": False, "ignore_merges": False, "vocab": vocab,
                  "merges": [f"{a} {b}" for a, b in merges]},
    }
    path = tmp_path / "tokenizer.json"
    path.write_text(json.dumps(payload, ensure_ascii=False), encoding="utf-8")
    theirs = hf.Tokenizer.from_file(str(path))
    ours = T.Tokenizer.tokenizer_json(str(path))
    assert ours.vocab_size == bos + 1
    for trial in range(300):
        text = random_text(rng, rng.randint(1, 60))
        want = theirs.encode(text).ids
        got = ours.encode(text)
        assert got == want, text
        assert ours.decode(got) == text        # special tokens are skipped, bytes restored
        assert theirs.decode(want) == text


# ---- SentencePiece merging against a plain restatement ----
def sp_encode_restated(pieces, max_len, text):
    """SentencePieceTokenizer.swift:68-112 over code points (the alphabet below has one code point per Character)."""
    ids = {p: i for i, (p, _) in enumerate(pieces)}
    tokens = []
    for ch in "▁" + text.replace(" ", "▁"):
        if ch in ids:
            tokens.append(ids[ch])
        else:
            tokens += [ids[f"<0x{b:02X}>"] for b in ch.encode("utf-8") if f"<0x{b:02X}>" in ids]
    while len(tokens) >= 2:
        best = None
        for i in range(len(tokens) - 1):
            merged = pieces[tokens[i]][0] + pieces[tokens[i + 1]][0]
            if len(merged.encode("utf-8")) <= max_len and merged in ids and (best is None or pieces[ids[merged]][1] > best[0]):
                best = (pieces[ids[merged]][1], i, ids[merged])
        if best is None:
            break
        tokens[best[1]:best[1] + 2] = [best[2]]
    return tokens


def test_sentencepiece_matches_restatement_on_random_text(tmp_path):
    rng = random.Random(3)
    letters = list("abcdeé中")
    pieces = [("▁", 0.0)] + [(c, 0.0) for c in letters] + [(f"<0x{b:02X}>", 0.0) for b in range(256)]
    seen = {p for p, _ in pieces}
    while len(pieces) < 400:
        a, b = rng.choice(pieces)[0], rng.choice(pieces)[0]
        if a.startswith("<0x") or b.startswith("<0x") or a + b in seen or len((a + b).encode()) > 12:
            continue
        seen.add(a + b)
        pieces.append((a + b, float(rng.randint(1, 6))))          # repeated scores: ties go to the leftmost pair
    (tmp_path / "tokenizer.bin").write_bytes(sp_model_bytes(pieces, max_token_length=10))
    tok = T.Tokenizer.sentencepiece(str(tmp_path / "tokenizer.bin"))
    alphabet = letters + [" ", " ", "x", "ß", "\n", "😀"]          # x, ß, newline, emoji: not pieces -> byte fallback
    for trial in range(300):
        text = "".join(rng.choice(alphabet) for _ in range(rng.randint(0, 30)))
        got = tok.encode(text)
        assert got == sp_encode_restated(pieces, 10, text), text
        assert tok.decode(got) == text     # the space decode drops (:140-144) is the mark encode put in front


def test_sentencepiece_characters_are_grapheme_clusters(tmp_path):
    # a Swift Character is a whole cluster: "e" + U+0301 is looked up as one piece, then falls back to its bytes
    pieces = [("▁", 0.0), ("e", 0.0), ("́", 0.0), ("é", 0.0)] + [(f"<0x{b:02X}>", 0.0) for b in range(256)]
    (tmp_path / "a.bin").write_bytes(sp_model_bytes(pieces))
    assert T.Tokenizer.sentencepiece(str(tmp_path / "a.bin")).encode("é") == [0, 3]
    (tmp_path / "b.bin").write_bytes(sp_model_bytes(pieces[:3] + pieces[4:]))
    ids = T.Tokenizer.sentencepiece(str(tmp_path / "b.bin")).encode("é\r\n")
    base = 3
    assert ids == [0] + [base + b for b in "é".encode()] + [base + 13, base + 10]   # "\r\n" is one Character too


def test_decode_repairs_invalid_utf8_and_ignores_unknown_ids(tmp_path):
    tok = T.Tokenizer.sentencepiece(make_sp_fixture(tmp_path, pieces=SP_PIECES + [("<0xE4>", 0.0), ("<0xB8>", 0.0), ("<0xAD>", 0.0)]))
    assert tok.decode([21, 22, 23]) == "中"
    assert tok.decode_bytes([21, 22, 1]) == "�H".encode()       # a truncated sequence is one replacement character
    assert tok.decode([1, 999, -1, 2]) == "He"
    g = T.Tokenizer.gpt2(*make_gpt2_fixture(tmp_path))
    assert g.decode([0, 77, 3]) == "Hello!"
