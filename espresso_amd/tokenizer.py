"""ctypes face of the tokenizers (declared in include/espresso_hip.h): the Tokenizer protocol of
Sources/ModelSupport/Tokenizer.swift (encode, decode, vocabSize) over the SentencePiece and byte-level
BPE implementations, and the engine's selection order."""
from __future__ import annotations

import ctypes as C

import numpy as np

from . import _lib

ERROR_NAMES = {
    0: "ok", 1: "unreadableFile",
    10: "truncatedModel", 11: "invalidMaxTokenLength", 12: "truncatedEntry", 13: "invalidUTF8Entry", 14: "emptyVocabulary",
    20: "malformedVocabulary", 21: "emptyVocabulary", 22: "nonContiguousTokenIDs", 23: "malformedTokenizerJSON",
    24: "unsupportedTokenizerModel", 25: "invalidPreTokenizerPattern", 30: "missingPath",
}


class TokenizerErrorStruct(C.Structure):
    _fields_ = [("code", C.c_int32), ("detail", C.c_int64), ("detail2", C.c_int64), ("text", C.c_char * 256)]


class TokenizerError(ValueError):
    """A case of SentencePieceTokenizerError / GPT2BPETokenizerError."""

    def __init__(self, code: int, detail: int, detail2: int, text: str):
        super().__init__(f"{ERROR_NAMES.get(code, code)}({detail}, {detail2}) {text}")
        self.code, self.case, self.detail, self.detail2, self.text = code, ERROR_NAMES.get(code, str(code)), detail, detail2, text


_declared = False


def _L():
    global _declared
    L = _lib.load_library()
    if _declared:
        return L
    vp, sz, cp = C.c_void_p, C.c_size_t, C.c_char_p
    for name, args in (("esp_tokenizer_load_sentencepiece", [cp]), ("esp_tokenizer_load_gpt2", [cp, cp]),
                       ("esp_tokenizer_load_tokenizer_json", [cp]), ("esp_tokenizer_load_dir", [vp, cp])):
        getattr(L, name).restype = vp
        getattr(L, name).argtypes = args
    L.esp_tokenizer_last_error.argtypes = [C.POINTER(TokenizerErrorStruct)]
    L.esp_tokenizer_free.argtypes = [vp]
    L.esp_tokenizer_vocab_size.restype = C.c_int; L.esp_tokenizer_vocab_size.argtypes = [vp]
    L.esp_tokenizer_kind.restype = cp; L.esp_tokenizer_kind.argtypes = [vp]
    L.esp_tokenizer_encode.restype = C.c_long; L.esp_tokenizer_encode.argtypes = [vp, cp, sz, vp, sz]
    L.esp_tokenizer_decode.restype = C.c_long; L.esp_tokenizer_decode.argtypes = [vp, vp, sz, vp, sz]
    L.esp_pretokenize.restype = C.c_long; L.esp_pretokenize.argtypes = [cp, cp, sz, vp, sz]
    _declared = True
    return L


def pretokenize(text: str, pattern: str | None = None) -> list[str]:
    """The chunks the byte-level BPE encodes one by one (text between matches is dropped)."""
    raw = text.encode("utf-8")
    pat = pattern.encode("utf-8") if pattern is not None else None
    n = _L().esp_pretokenize(pat, raw, len(raw), None, 0)
    if n < 0:
        raise _lib.EspressoError(int(n), _lib.last_error())
    out = np.zeros((max(n, 1), 2), dtype=np.int64)
    _L().esp_pretokenize(pat, raw, len(raw), out.ctypes.data_as(C.c_void_p), n)
    return [raw[a:b].decode("utf-8") for a, b in out[:n].tolist()]


class Tokenizer:
    def __init__(self, handle):
        if not handle:
            e = TokenizerErrorStruct()
            _L().esp_tokenizer_last_error(C.byref(e))
            raise TokenizerError(e.code, e.detail, e.detail2, e.text.decode(errors="replace"))
        self._h = handle

    # ---- constructors, named as the reference's initialisers ----
    @classmethod
    def sentencepiece(cls, model_path: str) -> "Tokenizer":
        return cls(_L().esp_tokenizer_load_sentencepiece(model_path.encode()))

    @classmethod
    def gpt2(cls, vocab_path: str, merges_path: str) -> "Tokenizer":
        return cls(_L().esp_tokenizer_load_gpt2(vocab_path.encode(), merges_path.encode()))

    @classmethod
    def tokenizer_json(cls, path: str) -> "Tokenizer":
        return cls(_L().esp_tokenizer_load_tokenizer_json(path.encode()))

    @classmethod
    def from_dir(cls, cfg, tokenizer_dir: str, architecture: str = "llama") -> "Tokenizer":
        from . import engine
        s = engine.config_struct(cfg)
        s.architecture = 0 if architecture == "gpt2" else 1
        return cls(_L().esp_tokenizer_load_dir(C.byref(s), tokenizer_dir.encode()))

    def close(self):
        if self._h:
            _L().esp_tokenizer_free(self._h)
            self._h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    @property
    def vocab_size(self) -> int:
        return _L().esp_tokenizer_vocab_size(self._h)

    @property
    def kind(self) -> str:
        return _L().esp_tokenizer_kind(self._h).decode()

    def encode(self, text: str) -> list[int]:
        raw = text.encode("utf-8", errors="surrogatepass")
        n = _L().esp_tokenizer_encode(self._h, raw, len(raw), None, 0)
        if n < 0:
            raise _lib.EspressoError(int(n), _lib.last_error())
        out = np.zeros(max(n, 1), dtype=np.int32)
        _L().esp_tokenizer_encode(self._h, raw, len(raw), out.ctypes.data_as(C.c_void_p), n)
        return out[:n].tolist()

    def decode_bytes(self, tokens) -> bytes:
        t = np.ascontiguousarray(tokens, dtype=np.int32)
        n = _L().esp_tokenizer_decode(self._h, t.ctypes.data_as(C.c_void_p), t.size, None, 0)
        if n < 0:
            raise _lib.EspressoError(int(n), _lib.last_error())
        buf = C.create_string_buffer(max(n, 1))
        _L().esp_tokenizer_decode(self._h, t.ctypes.data_as(C.c_void_p), t.size, buf, n)
        return buf.raw[:n]

    def decode(self, tokens) -> str:
        return self.decode_bytes(tokens).decode("utf-8")
