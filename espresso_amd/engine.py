"""ctypes face of the host layer: weight files, metadata, GGUF prepare, the engine and the exact
two-token harness (declared in include/espresso_hip.h)."""
from __future__ import annotations

import ctypes as C

import numpy as np

from . import _lib, llama


class ModelConfigStruct(C.Structure):
    _fields_ = [("name", C.c_char * 64)] + \
               [(n, C.c_int32) for n in ("n_layer", "n_head", "n_kv_head", "d_model", "head_dim", "hidden_dim", "vocab", "max_seq")] + \
               [("norm_eps", C.c_float), ("rope_theta", C.c_float), ("eos_token", C.c_int32), ("architecture", C.c_int32)]


class PrepareOptionsStruct(C.Structure):
    _fields_ = [("emit_dequantized_blobs", C.c_int32), ("emit_float32_sidecars", C.c_int32), ("qk_layout", C.c_int32)]


class GenerationResultStruct(C.Structure):
    _fields_ = [("token_count", C.c_int32), ("tokens_per_second", C.c_double), ("compile_time_ms", C.c_double),
                ("first_token_latency_ms", C.c_double), ("has_two_token_stats", C.c_int32),
                ("committed_exact_tokens_per_pass", C.c_double), ("accepted_future_tokens_per_pass", C.c_double),
                ("exact_head_backend", C.c_char * 48)]


class PromotionPlanStruct(C.Structure):
    _fields_ = [("committed_tokens", C.c_uint32 * 2), ("committed_exact_token_count", C.c_int32),
                ("accepted_future_token_count", C.c_int32), ("promoted_step_count", C.c_int32), ("next_current_token", C.c_uint32)]


class PassResultStruct(C.Structure):
    _fields_ = [("committed_tokens", C.c_uint32 * 2), ("committed_count", C.c_int32), ("next_current_token", C.c_uint32),
                ("proposer_latency_ms", C.c_double), ("verifier_trunk_latency_ms", C.c_double),
                ("verifier_logits_latency_ms", C.c_double), ("state_advance_latency_ms", C.c_double),
                ("accepted_future_token_count", C.c_int32), ("committed_exact_token_count", C.c_int32)]


RESET_FN = C.CFUNCTYPE(C.c_int, C.c_void_p)
PREFILL_FN = C.CFUNCTYPE(C.c_int, C.c_void_p, C.POINTER(C.c_uint32), C.c_int, C.POINTER(C.c_uint32))
PASS_FN = C.CFUNCTYPE(C.c_int, C.c_void_p, C.c_uint32, C.c_int, C.POINTER(PassResultStruct))


class ExactTwoTokenModelStruct(C.Structure):
    _fields_ = [("context", C.c_void_p), ("reset", RESET_FN), ("prefill_selected_token", PREFILL_FN),
                ("perform_exact_two_token_pass", PASS_FN)]


_declared = False


def _L():
    global _declared
    L = _lib.load_library()
    if _declared:
        return L
    vp, sz, i32, cp = C.c_void_p, C.c_size_t, C.c_int, C.c_char_p
    L.esp_weight_blob_bytes.restype = sz; L.esp_weight_blob_bytes.argtypes = [sz]
    L.esp_weight_blob_build.restype = i32; L.esp_weight_blob_build.argtypes = [vp, sz, vp]
    L.esp_blob_weight_load.restype = C.c_long; L.esp_blob_weight_load.argtypes = [cp, vp, sz]
    L.esp_layer_weight_path.restype = i32; L.esp_layer_weight_path.argtypes = [i32, cp, i32, cp, sz]
    L.esp_model_config_load_metadata.restype = i32; L.esp_model_config_load_metadata.argtypes = [cp, C.POINTER(ModelConfigStruct)]
    L.esp_model_config_write_metadata.restype = i32; L.esp_model_config_write_metadata.argtypes = [C.POINTER(ModelConfigStruct), cp]
    L.esp_gguf_prepare.restype = i32
    L.esp_gguf_prepare.argtypes = [cp, cp, C.POINTER(PrepareOptionsStruct), C.POINTER(ModelConfigStruct), C.POINTER(i32)]
    L.esp_engine_build.restype = vp
    L.esp_engine_build.argtypes = [C.POINTER(ModelConfigStruct), cp, cp, C.POINTER(cp), C.POINTER(cp), i32]
    L.esp_engine_free.argtypes = [vp]
    L.esp_engine_runtime.restype = vp; L.esp_engine_runtime.argtypes = [vp]
    L.esp_engine_generate.restype = i32
    L.esp_engine_generate.argtypes = [vp, vp, i32, i32, C.c_float, C.POINTER(cp), C.POINTER(cp), i32, vp, C.POINTER(GenerationResultStruct)]
    L.esp_engine_generate_text.restype = i32
    L.esp_engine_generate_text.argtypes = [vp, cp, sz, i32, C.c_float, C.POINTER(cp), C.POINTER(cp), i32, vp, vp, sz, C.POINTER(sz),
                                           C.POINTER(GenerationResultStruct)]
    L.esp_exact_two_token_promotion_plan.argtypes = [C.c_uint32] * 4 + [i32, C.POINTER(PromotionPlanStruct)]
    L.esp_exact_two_token_harness_generate.restype = i32
    L.esp_exact_two_token_harness_generate.argtypes = [C.POINTER(ExactTwoTokenModelStruct), vp, vp, vp, i32, i32, vp, C.POINTER(i32), vp, vp, C.POINTER(i32)]
    _declared = True
    return L


def _ptr(a):
    return a.ctypes.data_as(C.c_void_p)


def config_struct(cfg: llama.MultiModelConfig) -> ModelConfigStruct:
    return ModelConfigStruct(cfg.name.encode()[:63], cfg.n_layer, cfg.n_head, cfg.n_kv_head, cfg.d_model, cfg.head_dim, cfg.hidden_dim,
                             cfg.vocab, cfg.max_seq, cfg.norm_eps, cfg.rope_theta, cfg.eos_token, 0 if cfg.architecture == "gpt2" else 1)


def config_from_struct(s: ModelConfigStruct) -> llama.MultiModelConfig:
    return llama.MultiModelConfig(n_layer=s.n_layer, n_head=s.n_head, n_kv_head=s.n_kv_head, d_model=s.d_model, head_dim=s.head_dim,
                                  hidden_dim=s.hidden_dim, vocab=s.vocab, max_seq=s.max_seq, norm_eps=s.norm_eps,
                                  rope_theta=s.rope_theta, eos_token=s.eos_token, name=s.name.decode(),
                                  architecture="gpt2" if s.architecture == 0 else "llama")


# ---- registry and head strategy ----------------------------------------------
def model_registry() -> dict:
    """ModelRegistry.all: {name: config}."""
    L = _L()
    out = {}
    for i in range(L.esp_model_registry_count()):
        s = ModelConfigStruct()
        _lib.check(L.esp_model_registry_at(i, C.byref(s)))
        out[s.name.decode()] = config_from_struct(s)
    return out


def model_registry_config(name: str):
    """ModelRegistry.config(named:): None when unknown."""
    s = ModelConfigStruct()
    return config_from_struct(s) if _L().esp_model_registry_config(name.encode(), C.byref(s)) == 0 else None


CLASSIFIER_STRATEGIES = ("ane", "cpuPartitionedFP32", "cpuFP16Tiled")


def classifier_strategy(cfg: llama.MultiModelConfig, has_exact_float32_lm_head: bool = False) -> tuple[str, str]:
    """ClassifierStrategy.select -> (case name, exactHeadBackendLabel)."""
    L = _L()
    L.esp_classifier_strategy_select.restype = C.c_int
    s, label = config_struct(cfg), C.create_string_buffer(48)
    k = L.esp_classifier_strategy_select(C.byref(s), int(has_exact_float32_lm_head), label, C.c_size_t(48))
    if k < 0:
        raise _lib.EspressoError(k, _lib.last_error())
    return CLASSIFIER_STRATEGIES[k], label.value.decode()


# ---- weight files -----------------------------------------------------------
def weight_blob_build(weights) -> bytes:
    w = np.ascontiguousarray(weights, dtype=np.float32).ravel()
    out = np.zeros(int(_L().esp_weight_blob_bytes(w.size)), dtype=np.uint8)
    _lib.check(_L().esp_weight_blob_build(_ptr(w), w.size, _ptr(out)))
    return out.tobytes()


def blob_weight_load(path: str):
    """Returns (count_or_negative_error, values)."""
    n = _L().esp_blob_weight_load(path.encode(), None, 0)
    if n < 0:
        return int(n), None
    out = np.empty(n, dtype=np.float32)
    _L().esp_blob_weight_load(path.encode(), _ptr(out), n)
    return int(n), out


def layer_weight_path(layer: int, blob_dir: str, slot: int) -> str:
    buf = C.create_string_buffer(4096)
    n = _L().esp_layer_weight_path(layer, blob_dir.encode(), slot, buf, 4096)
    if n < 0:
        raise _lib.EspressoError(n, _lib.last_error())
    return buf.value.decode()


def load_metadata(path: str) -> llama.MultiModelConfig:
    s = ModelConfigStruct()
    _lib.check(_L().esp_model_config_load_metadata(path.encode(), C.byref(s)))
    return config_from_struct(s)


def write_metadata(cfg: llama.MultiModelConfig, path: str) -> None:
    s = config_struct(cfg)
    _lib.check(_L().esp_model_config_write_metadata(C.byref(s), path.encode()))


# ---- GGUF ---------------------------------------------------------------------
def gguf_prepare(gguf_path: str, output_dir: str, emit_dequantized_blobs=False, emit_float32_sidecars=True, qk_layout=-1):
    """GGUFModelLoader.prepare -> (config, weight_dir, tensor_count)."""
    opt = PrepareOptionsStruct(int(emit_dequantized_blobs), int(emit_float32_sidecars), qk_layout)
    s, n = ModelConfigStruct(), C.c_int(0)
    _lib.check(_L().esp_gguf_prepare(gguf_path.encode(), output_dir.encode(), C.byref(opt), C.byref(s), C.byref(n)))
    return config_from_struct(s), output_dir, n.value


class PrepareCacheOptionsStruct(C.Structure):
    _fields_ = [("cache_enabled", C.c_int32), ("sidecar_mode", C.c_int32), ("cache_root", C.c_char * 1024),
                ("selected_sidecars", C.c_char * 2048)]


SIDECAR_MODES = ("automatic", "none", "essential", "selected", "full")


class PrepareOptions:
    """GGUFModelLoader.PrepareOptions: artifact cache mode, cache root, exact-float32 sidecar mode."""

    def __init__(self, artifact_cache_enabled=True, cache_root=None, sidecar_mode="automatic", selected_sidecars=()):
        self.artifact_cache_enabled = artifact_cache_enabled
        self.cache_root = cache_root
        self.sidecar_mode = sidecar_mode
        self.selected_sidecars = set(selected_sidecars)

    @classmethod
    def environment(cls, environment: dict):
        """PrepareOptions.environment(_:)."""
        L = _L()
        L.esp_gguf_prepare_options_from_environment.restype = C.c_int
        k, v, n = _env_arrays(environment)
        s = PrepareCacheOptionsStruct()
        _lib.check(L.esp_gguf_prepare_options_from_environment(k, v, n, C.byref(s)))
        names = [x for x in s.selected_sidecars.decode().split(",") if x]
        return cls(bool(s.cache_enabled), s.cache_root.decode() or None, SIDECAR_MODES[s.sidecar_mode], names)

    def struct(self) -> PrepareCacheOptionsStruct:
        return PrepareCacheOptionsStruct(int(self.artifact_cache_enabled), SIDECAR_MODES.index(self.sidecar_mode),
                                         (self.cache_root or "").encode(), ",".join(sorted(self.selected_sidecars)).encode())


def gguf_artifact_cache_key(gguf_path: str, options: PrepareOptions, environment: dict | None = None) -> str:
    """GGUFModelLoader.artifactCacheKey."""
    L = _L()
    L.esp_gguf_artifact_cache_key.restype = C.c_int
    k, v, n = _env_arrays(environment)
    s, out = options.struct(), C.create_string_buffer(80)
    _lib.check(L.esp_gguf_artifact_cache_key(gguf_path.encode(), C.byref(s), k, v, n, out, C.c_size_t(80)))
    return out.value.decode()


def gguf_prepare_cached(gguf_path: str, options: PrepareOptions, environment: dict | None = None, emit_dequantized_blobs=False,
                        emit_float32_sidecars=True, qk_layout=-1):
    """GGUFModelLoader.prepare(ggufURL:options:) -> (config, weight_dir, tensor_count); the directory is chosen by the cache."""
    L = _L()
    L.esp_gguf_prepare_cached.restype = C.c_int
    k, v, n = _env_arrays(environment)
    s, conv = options.struct(), PrepareOptionsStruct(int(emit_dequantized_blobs), int(emit_float32_sidecars), qk_layout)
    cfg, count, out = ModelConfigStruct(), C.c_int(0), C.create_string_buffer(4096)
    _lib.check(L.esp_gguf_prepare_cached(gguf_path.encode(), C.byref(s), C.byref(conv), k, v, n, C.byref(cfg), C.byref(count), out,
                                         C.c_size_t(4096)))
    return config_from_struct(cfg), out.value.decode(), count.value


def gguf_cleanup(weight_dir: str) -> None:
    """GGUFModelLoader.cleanup(weightDir:): managed cache directories are kept."""
    L = _L()
    L.esp_gguf_cleanup.restype = C.c_int
    _lib.check(L.esp_gguf_cleanup(weight_dir.encode()))


def gguf_default_cache_root() -> str:
    L = _L()
    L.esp_gguf_default_cache_root.restype = C.c_int
    out = C.create_string_buffer(4096)
    _lib.check(L.esp_gguf_default_cache_root(out, C.c_size_t(4096)))
    return out.value.decode()


class RunGGUFInfoStruct(C.Structure):
    _fields_ = [("config", ModelConfigStruct), ("tensor_count", C.c_int32), ("kept_weight_dir", C.c_int32), ("prepare_ms", C.c_double),
                ("build_ms", C.c_double), ("weight_dir", C.c_char * 1024)]


def run_gguf(gguf_path: str, tokenizer_dir: str, prompt: str, max_tokens: int = 32, environment: dict | None = None) -> dict:
    """RunGGUF.main: prepare -> build -> generate(prompt) -> cleanup.  Returns text, tokens, the generation figures and
    what was prepared (config, tensor count, times, the weight directory and whether it was kept)."""
    L = _L()
    L.esp_run_gguf.restype = C.c_int
    k, v, n = _env_arrays(environment)
    p = prompt.encode()
    toks = (C.c_uint32 * max(max_tokens, 1))()
    text = C.create_string_buffer(1 << 20)
    nbytes, res, info = C.c_size_t(0), GenerationResultStruct(), RunGGUFInfoStruct()
    _lib.check(L.esp_run_gguf(gguf_path.encode(), tokenizer_dir.encode(), p, C.c_size_t(len(p)), max_tokens, k, v, n, toks, text,
                              C.c_size_t(len(text)), C.byref(nbytes), C.byref(res), C.byref(info)))
    return {"text": text.raw[:min(nbytes.value, len(text))].decode("utf-8", "replace"), "tokens": list(toks[:res.token_count]),
            "tokens_per_second": res.tokens_per_second, "compile_time_ms": res.compile_time_ms,
            "first_token_latency_ms": res.first_token_latency_ms, "config": config_from_struct(info.config),
            "tensor_count": info.tensor_count, "prepare_ms": info.prepare_ms, "build_ms": info.build_ms,
            "weight_dir": info.weight_dir.decode(), "kept_weight_dir": bool(info.kept_weight_dir)}


# ---- engine ---------------------------------------------------------------------
def _env_arrays(env: dict | None):
    env = env or {}
    keys = (C.c_char_p * max(len(env), 1))(*[k.encode() for k in env])
    vals = (C.c_char_p * max(len(env), 1))(*[v.encode() for v in env.values()])
    return keys, vals, len(env)


class RealModelInferenceEngine:
    """RealModelInferenceEngine.build / generate (token-id form)."""

    def __init__(self, cfg: llama.MultiModelConfig, weight_dir: str, tokenizer_dir: str | None = None, environment: dict | None = None):
        self.cfg = cfg
        s = config_struct(cfg)
        k, v, n = _env_arrays(environment)
        self._h = _L().esp_engine_build(C.byref(s), weight_dir.encode(), tokenizer_dir.encode() if tokenizer_dir else None, k, v, n)
        if not self._h:
            raise _lib.EspressoError(-1, _lib.last_error())

    def close(self):
        if self._h:
            _L().esp_engine_free(self._h)
            self._h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def generate(self, prompt_tokens, max_tokens: int, temperature: float = 0.0, environment: dict | None = None):
        p = np.ascontiguousarray(prompt_tokens, dtype=np.uint32)
        out = np.zeros(max(max_tokens, 1), dtype=np.uint32)
        r = GenerationResultStruct()
        k, v, n = _env_arrays(environment)
        _lib.check(_L().esp_engine_generate(self._h, _ptr(p), p.size, max_tokens, C.c_float(temperature), k, v, n, _ptr(out), C.byref(r)))
        res = {f: getattr(r, f) for f, _ in r._fields_}
        res["exact_head_backend"] = r.exact_head_backend.decode()
        return out[:r.token_count].tolist(), res

    def generate_text(self, prompt: str, max_tokens: int, temperature: float = 0.0, environment: dict | None = None):
        """generate(prompt:maxTokens:temperature:) -> (text of prompt + generated tokens, generated tokens, result fields)."""
        raw = prompt.encode("utf-8")
        out = np.zeros(max(max_tokens, 1), dtype=np.uint32)
        r = GenerationResultStruct()
        k, v, n = _env_arrays(environment)
        cap = 1 << 20
        buf, nbytes = C.create_string_buffer(cap), C.c_size_t(0)
        _lib.check(_L().esp_engine_generate_text(self._h, raw, len(raw), max_tokens, C.c_float(temperature), k, v, n, _ptr(out), buf, cap,
                                                 C.byref(nbytes), C.byref(r)))
        res = {f: getattr(r, f) for f, _ in r._fields_}
        res["exact_head_backend"] = r.exact_head_backend.decode()
        return buf.raw[:min(nbytes.value, cap)].decode("utf-8", errors="replace"), out[:r.token_count].tolist(), res

    def runtime(self) -> llama.LlamaRuntime:
        """A non-owning view of the engine's runtime."""
        rt = llama.LlamaRuntime.__new__(llama.LlamaRuntime)
        rt.cfg, rt._L, rt._h = self.cfg, _L(), _L().esp_engine_runtime(self._h)
        rt.close = lambda: None
        return rt


def sample_token(logits, temperature: float, unit: float) -> int:
    x = np.ascontiguousarray(logits, dtype=np.float32)
    L = _L()
    L.esp_sample_token.restype = C.c_int
    L.esp_sample_token.argtypes = [C.c_void_p, C.c_int, C.c_float, C.c_double]
    r = L.esp_sample_token(_ptr(x), x.size, temperature, unit)
    if r < 0:
        raise _lib.EspressoError(r, _lib.last_error())
    return r


def splitmix64_units(seed: int, count: int) -> list[float]:
    L = _L()
    L.esp_splitmix64_unit.restype = C.c_double
    L.esp_splitmix64_unit.argtypes = [C.POINTER(C.c_uint64)]
    state = C.c_uint64(seed)
    return [L.esp_splitmix64_unit(C.byref(state)) for _ in range(count)]


# ---- exact two-token harness -----------------------------------------------------
def promotion_plan(current, proposed, exact_next, exact_future, budget) -> dict:
    p = PromotionPlanStruct()
    _L().esp_exact_two_token_promotion_plan(current, proposed, exact_next, exact_future, budget, C.byref(p))
    return {"committed_tokens": list(p.committed_tokens)[:p.committed_exact_token_count], "next_current_token": p.next_current_token,
            "committed_exact_token_count": p.committed_exact_token_count, "accepted_future_token_count": p.accepted_future_token_count,
            "promoted_step_count": p.promoted_step_count}


def harness_generate(prompt_tokens, max_new_tokens: int, model: ExactTwoTokenModelStruct | None = None,
                     target: llama.LlamaRuntime | None = None, draft: llama.LlamaRuntime | None = None):
    """ExactTwoTokenGenerationHarness.generate -> (tokens, committed per pass, accepted per pass)."""
    p = np.ascontiguousarray(prompt_tokens, dtype=np.uint32)
    cap = max(max_new_tokens, 1)
    out = np.zeros(cap + 1, dtype=np.uint32)
    com, acc = np.zeros(cap, dtype=np.int32), np.zeros(cap, dtype=np.int32)
    n, passes = C.c_int(0), C.c_int(0)
    _lib.check(_L().esp_exact_two_token_harness_generate(C.byref(model) if model is not None else None,
                                                         target._h if target is not None else None,
                                                         draft._h if draft is not None else None,
                                                         _ptr(p), p.size, max_new_tokens, _ptr(out), C.byref(n), _ptr(com), _ptr(acc),
                                                         C.byref(passes)))
    return out[:n.value].tolist(), com[:passes.value].tolist(), acc[:passes.value].tolist()
