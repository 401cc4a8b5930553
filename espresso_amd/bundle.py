"""ctypes face of the .esp bundle bridge (declared in include/espresso_hip.h): ESPManifest.parseTOML / renderTOML,
ESPBundleArchive.open with its SHA-256 catalog, ESPRuntimeResolver.selectBackend and ESPRuntimeRunner.generate."""
from __future__ import annotations

import ctypes as C

import numpy as np

from . import _lib, engine

ERROR_NAMES = {
    0: "ok", 1: "emptyField", 2: "invalidMaxContext", 3: "invalidContextTarget", 4: "invalidAdapterSlots", 5: "missingBackends",
    6: "missingProfiles", 7: "invalidWeightBits", 8: "invalidActivationBits", 9: "missingTopLevelEntry", 10: "missingManifest",
    11: "malformedLine", 12: "malformedSection", 13: "unsupportedValue", 14: "invalidOutputHead", 15: "invalidDraft",
    16: "invalidReferencedPath", 17: "missingReferencedFile", 18: "signatureMismatch", 19: "unreadableFile",
    30: "noCompatibleBackend", 31: "noCompatibleProfile", 32: "requestedContextExceedsTarget",
}

REQUIRED_TOP_LEVEL_ENTRIES = ["arch", "tokenizer", "weights", "graphs", "states", "adapters", "compiled", "benchmarks", "licenses", "signatures"]


class BundleErrorStruct(C.Structure):
    _fields_ = [("code", C.c_int32), ("detail", C.c_int64), ("detail2", C.c_int64), ("text", C.c_char * 256)]


class SelectionStruct(C.Structure):
    _fields_ = [("backend", C.c_char * 16), ("profile", C.c_char * 16), ("context_target_tokens", C.c_int64),
                ("has_output_head", C.c_int32), ("has_draft", C.c_int32), ("reason", C.c_char * 64)]


class BundleError(ValueError):
    """A case of ESPBundleValidationError / ESPRuntimeSelectionError."""

    def __init__(self, code, detail, detail2, text):
        super().__init__(f"{ERROR_NAMES.get(code, code)}({detail}, {detail2}) {text}")
        self.code, self.case, self.detail, self.detail2, self.text = code, ERROR_NAMES.get(code, str(code)), detail, detail2, text


_declared = False


def _L():
    global _declared
    L = _lib.load_library()
    if _declared:
        return L
    vp, sz, cp, i32 = C.c_void_p, C.c_size_t, C.c_char_p, C.c_int
    L.esp_bundle_last_error.argtypes = [C.POINTER(BundleErrorStruct)]
    L.esp_manifest_parse_toml.restype = i32; L.esp_manifest_parse_toml.argtypes = [cp, sz, vp, sz, C.POINTER(sz)]
    L.esp_bundle_write_signature_catalog.restype = i32; L.esp_bundle_write_signature_catalog.argtypes = [cp]
    L.esp_bundle_open.restype = vp; L.esp_bundle_open.argtypes = [cp, i32]
    L.esp_bundle_free.argtypes = [vp]
    L.esp_bundle_model_config.restype = i32; L.esp_bundle_model_config.argtypes = [vp, C.POINTER(engine.ModelConfigStruct)]
    L.esp_bundle_resolve.restype = i32; L.esp_bundle_resolve.argtypes = [vp, C.c_long, i32, C.POINTER(SelectionStruct)]
    L.esp_bundle_environment_overrides.restype = C.c_long; L.esp_bundle_environment_overrides.argtypes = [vp, C.c_long, i32, vp, sz]
    L.esp_bundle_generate.restype = i32
    L.esp_bundle_generate.argtypes = [vp, cp, sz, i32, C.c_float, C.POINTER(cp), C.POINTER(cp), i32, vp, vp, sz, C.POINTER(sz),
                                      C.POINTER(engine.GenerationResultStruct), C.POINTER(SelectionStruct)]
    _declared = True
    return L


def _raise_last(rc=None):
    e = BundleErrorStruct()
    _L().esp_bundle_last_error(C.byref(e))
    if e.code != 0:
        raise BundleError(e.code, e.detail, e.detail2, e.text.decode(errors="replace"))
    raise _lib.EspressoError(rc if rc is not None else -1, _lib.last_error())


def parse_manifest(text: str) -> str:
    """ESPManifest.parseTOML(text).renderTOML()"""
    raw = text.encode()
    n = C.c_size_t(0)
    buf = C.create_string_buffer(1 << 16)
    rc = _L().esp_manifest_parse_toml(raw, len(raw), buf, len(buf), C.byref(n))
    if rc != 0:
        _raise_last(rc)
    return buf.raw[:n.value].decode()


def write_signature_catalog(bundle_dir: str) -> None:
    rc = _L().esp_bundle_write_signature_catalog(bundle_dir.encode())
    if rc != 0:
        _raise_last(rc)


def _selection(s: SelectionStruct) -> dict:
    return {"backend": s.backend.decode(), "profile": s.profile.decode(), "context_target_tokens": s.context_target_tokens,
            "has_output_head": bool(s.has_output_head), "has_draft": bool(s.has_draft), "reason": s.reason.decode()}


class RuntimeBundle:
    """ESPRuntimeBundle.open(at:)"""

    def __init__(self, bundle_dir: str, verify_signatures: bool = True):
        self._h = _L().esp_bundle_open(bundle_dir.encode(), int(verify_signatures))
        if not self._h:
            _raise_last()

    def close(self):
        if self._h:
            _L().esp_bundle_free(self._h)
            self._h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    @property
    def config(self):
        s = engine.ModelConfigStruct()
        _lib.check(_L().esp_bundle_model_config(self._h, C.byref(s)))
        return engine.config_from_struct(s)

    def resolve(self, requested_context_tokens: int | None = None, supports_ane_private: bool = True) -> dict:
        s = SelectionStruct()
        rc = _L().esp_bundle_resolve(self._h, -1 if requested_context_tokens is None else requested_context_tokens, int(supports_ane_private), C.byref(s))
        if rc != 0:
            _raise_last(rc)
        return _selection(s)

    def environment_overrides(self, requested_context_tokens: int | None = None, supports_ane_private: bool = True) -> dict:
        buf = C.create_string_buffer(1 << 14)
        n = _L().esp_bundle_environment_overrides(self._h, -1 if requested_context_tokens is None else requested_context_tokens,
                                                  int(supports_ane_private), buf, len(buf))
        if n < 0:
            _raise_last(int(n))
        return dict(line.split("=", 1) for line in buf.raw[:n].decode().splitlines())

    def generate(self, prompt: str, max_tokens: int, temperature: float = 0.0, environment: dict | None = None):
        """ESPRuntimeRunner.generate -> (text, generated tokens, result fields, selection)."""
        raw = prompt.encode()
        out = np.zeros(max(max_tokens, 1), dtype=np.uint32)
        r, sel = engine.GenerationResultStruct(), SelectionStruct()
        k, v, n = engine._env_arrays(environment)
        cap = 1 << 20
        buf, nbytes = C.create_string_buffer(cap), C.c_size_t(0)
        rc = _L().esp_bundle_generate(self._h, raw, len(raw), max_tokens, C.c_float(temperature), k, v, n, out.ctypes.data_as(C.c_void_p),
                                      buf, cap, C.byref(nbytes), C.byref(r), C.byref(sel))
        if rc != 0:
            _raise_last(rc)
        res = {f: getattr(r, f) for f, _ in r._fields_}
        res["exact_head_backend"] = r.exact_head_backend.decode()
        return buf.raw[:min(nbytes.value, cap)].decode("utf-8", errors="replace"), out[:r.token_count].tolist(), res, _selection(sel)
