"""ctypes face of the GPU-resident llama runtime (ESPLlamaRuntime in include/espresso_hip.h)."""
from __future__ import annotations

import ctypes as C
from dataclasses import dataclass

import numpy as np

from . import _lib

SLOT_TOKEN_EMBEDDING, SLOT_FINAL_NORM, SLOT_LM_HEAD = 0, 1, 2
SLOT_RMS_ATT, SLOT_WQ, SLOT_WK, SLOT_WV, SLOT_WO, SLOT_RMS_FFN, SLOT_W1, SLOT_W2, SLOT_W3, SLOT_Q_NORM, SLOT_K_NORM = range(10, 21)
LAYER_SLOTS = {"rms_att": SLOT_RMS_ATT, "wq": SLOT_WQ, "wk": SLOT_WK, "wv": SLOT_WV, "wo": SLOT_WO,
               "rms_ffn": SLOT_RMS_FFN, "w1": SLOT_W1, "w2": SLOT_W2, "w3": SLOT_W3,
               "q_norm": SLOT_Q_NORM, "k_norm": SLOT_K_NORM}


@dataclass
class MultiModelConfig:
    """Sources/ModelSupport/MultiModelConfig.swift:3-55 (llama architecture)."""
    n_layer: int
    n_head: int
    n_kv_head: int
    d_model: int
    head_dim: int
    hidden_dim: int
    vocab: int
    max_seq: int
    norm_eps: float = 1e-5
    rope_theta: float = 10000.0
    eos_token: int = -1
    name: str = "llama"
    architecture: str = "llama"   # or "gpt2" (registry entries only: the runtime runs the llama family)

    @property
    def attention_dim(self) -> int:
        return self.n_head * self.head_dim

    @property
    def kv_dim(self) -> int:
        return self.n_kv_head * self.head_dim


def _ptr(a: np.ndarray):
    return a.ctypes.data_as(C.c_void_p)


class LlamaRuntime:
    def __init__(self, cfg: MultiModelConfig, kv_format: int = _lib.FORMAT_F32, max_sequences: int = 1):
        self.cfg = cfg
        self._L = _lib.load_library()
        c = _lib.LlamaConfigStruct(cfg.n_layer, cfg.n_head, cfg.n_kv_head, cfg.d_model, cfg.head_dim, cfg.hidden_dim,
                                   cfg.vocab, cfg.max_seq, cfg.norm_eps, cfg.rope_theta, cfg.eos_token, kv_format,
                                   max_sequences)
        self._h = self._L.esp_llama_create(C.byref(c))
        if not self._h:
            raise _lib.EspressoError(-1, _lib.last_error())

    def close(self) -> None:
        if self._h:
            self._L.esp_llama_free(self._h)
            self._h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def set_weight(self, layer: int, slot: int, fmt: int, data: np.ndarray) -> None:
        a = np.ascontiguousarray(data)
        raw = a.view(np.uint8).ravel()
        _lib.check(self._L.esp_llama_set_weight(self._h, layer, slot, fmt, _ptr(raw), raw.size))

    def finalize(self) -> None:
        _lib.check(self._L.esp_llama_finalize(self._h))

    @property
    def weight_bytes(self) -> int:
        return int(self._L.esp_llama_weight_bytes(self._h))

    @property
    def resident_weight_bytes(self) -> int:
        return int(self._L.esp_llama_resident_weight_bytes(self._h))

    def reset(self) -> None:
        _lib.check(self._L.esp_llama_reset(self._h))

    def prefill(self, tokens, sequence: int = 0) -> None:
        t = np.ascontiguousarray(tokens, dtype=np.uint32)
        _lib.check(self._L.esp_llama_prefill(self._h, sequence, _ptr(t), t.size))

    def advance(self, token: int, sequence: int = 0) -> None:
        _lib.check(self._L.esp_llama_advance(self._h, sequence, C.c_uint32(token)))

    def select_greedy(self, sequence: int = 0) -> int:
        t = C.c_uint32(0)
        _lib.check(self._L.esp_llama_select_greedy_token(self._h, sequence, C.byref(t)))
        return int(t.value)

    def visible(self, sequence: int = 0) -> int:
        return int(self._L.esp_llama_visible_token_count(self._h, sequence))

    def set_visible(self, count: int, sequence: int = 0) -> None:
        _lib.check(self._L.esp_llama_set_visible_token_count(self._h, sequence, count))

    def last_hidden(self, sequence: int = 0) -> np.ndarray:
        out = np.empty(self.cfg.d_model, dtype=np.float32)
        _lib.check(self._L.esp_llama_read_last_hidden(self._h, sequence, _ptr(out)))
        return out

    def logits(self, sequence: int = 0) -> np.ndarray:
        out = np.empty(self.cfg.vocab, dtype=np.float32)
        _lib.check(self._L.esp_llama_read_logits(self._h, sequence, _ptr(out)))
        return out

    def generate(self, prompt, max_tokens: int):
        p = np.ascontiguousarray(prompt, dtype=np.uint32)
        out = np.zeros(max(max_tokens, 1), dtype=np.uint32)
        lat = np.zeros(max(max_tokens, 1), dtype=np.float64)
        n = C.c_int(0)
        st = _lib.GenerationStatsStruct()
        _lib.check(self._L.esp_llama_generate(self._h, _ptr(p), p.size, max_tokens, _ptr(out), C.byref(n), C.byref(st), _ptr(lat)))
        stats = {k: getattr(st, k) for k, _ in st._fields_}
        stats["token_latencies_ms"] = lat[:n.value].tolist()
        return out[:n.value].tolist(), stats


def generate_two_token(target: LlamaRuntime, draft: LlamaRuntime, prompt, max_tokens: int, reference_accounting: bool = True):
    L = _lib.load_library()
    p = np.ascontiguousarray(prompt, dtype=np.uint32)
    out = np.zeros(max(max_tokens, 1), dtype=np.uint32)
    n = C.c_int(0)
    st, tt = _lib.GenerationStatsStruct(), _lib.TwoTokenStatsStruct()
    _lib.check(L.esp_llama_generate_two_token(target._h, draft._h, _ptr(p), p.size, max_tokens, int(reference_accounting),
                                              _ptr(out), C.byref(n), C.byref(st), C.byref(tt)))
    stats = {k: getattr(st, k) for k, _ in st._fields_}
    stats.update({k: getattr(tt, k) for k, _ in tt._fields_})
    return out[:n.value].tolist(), stats


def generate_batch(target: LlamaRuntime, prompts, max_tokens: int, draft: LlamaRuntime | None = None):
    """Lock-step greedy decode of len(prompts) sequences; with `draft`, the exact two-token loop over all of them.
    Returns (list of token lists, stats)."""
    L = _lib.load_library()
    L.esp_llama_generate_batch.restype = C.c_int
    n = len(prompts)
    arrays = [np.ascontiguousarray(p, dtype=np.uint32) for p in prompts]
    ptrs = (C.c_void_p * n)(*[a.ctypes.data for a in arrays])
    counts = (C.c_int * n)(*[a.size for a in arrays])
    out = np.zeros((n, max(max_tokens, 1)), dtype=np.uint32)
    out_counts = (C.c_int * n)()
    tt = _lib.TwoTokenStatsStruct()
    ms = C.c_double(0)
    L.esp_llama_generate_batch.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_int, C.c_int, C.c_void_p, C.c_void_p,
                                           C.c_void_p, C.POINTER(C.c_double)]
    _lib.check(L.esp_llama_generate_batch(target._h, draft._h if draft is not None else None, ptrs, counts, n, max_tokens, _ptr(out),
                                          out_counts, C.byref(tt), C.byref(ms)))
    stats = {"decode_ms": ms.value, "passes": tt.passes, "committed_total": tt.committed_total, "accepted_total": tt.accepted_total}
    return [out[s, :out_counts[s]].tolist() for s in range(n)], stats


def load_packed_weights(rt: LlamaRuntime, packed: dict, matrix_format: int, embedding_format: int = _lib.FORMAT_F16,
                        norm_format: int = _lib.FORMAT_F16) -> None:
    """packed: {"embedding", "final_norm", "lm_head", "layers": [{"rms_att", "wq", ...}]} of raw GGUF-layout bytes."""
    rt.set_weight(0, SLOT_TOKEN_EMBEDDING, embedding_format, packed["embedding"])
    rt.set_weight(0, SLOT_FINAL_NORM, norm_format, packed["final_norm"])
    rt.set_weight(0, SLOT_LM_HEAD, matrix_format, packed["lm_head"])
    for l, layer in enumerate(packed["layers"]):
        for name, data in layer.items():
            is_matrix = name in ("wq", "wk", "wv", "wo", "w1", "w2", "w3")
            rt.set_weight(l, LAYER_SLOTS[name], matrix_format if is_matrix else norm_format, data)
    rt.finalize()


KERNEL_CLASSES = ("qkv", "wo", "gate_up", "down", "head", "attention", "event_pair")


def continue_greedy(rt: LlamaRuntime, steps: int, sequence: int = 0) -> list[int]:
    out = np.zeros(max(steps, 1), dtype=np.uint32)
    _lib.check(rt._L.esp_llama_continue_greedy(rt._h, sequence, steps, _ptr(out)))
    return out[:steps].tolist()


def set_graph_replay(rt: LlamaRuntime, enabled: bool) -> None:
    _lib.check(rt._L.esp_llama_set_graph_replay(rt._h, int(enabled)))


def set_merged_attention(rt: LlamaRuntime, enabled: bool) -> bool:
    """Returns whether the one-launch attention merged by the wo GEMV is in use after the call."""
    r = rt._L.esp_llama_set_merged_attention(rt._h, int(enabled))
    if r < 0:
        _lib.check(r)
    return bool(r)


def set_split_activations(rt: LlamaRuntime, enabled: bool) -> None:
    _lib.check(rt._L.esp_llama_set_split_activations(rt._h, int(enabled)))


def set_matrix_prefill(rt: LlamaRuntime, enabled: bool) -> None:
    _lib.check(rt._L.esp_llama_set_matrix_prefill(rt._h, int(enabled)))


def set_kernel_timing(rt: LlamaRuntime, enabled: bool) -> None:
    _lib.check(rt._L.esp_llama_set_kernel_timing(rt._h, int(enabled)))


def time_kernel(rt: LlamaRuntime, name: str, iters: int = 8) -> float:
    """Mean microseconds of back-to-back launches of one GEMV class over all layers (invalidates sequence state)."""
    rt._L.esp_llama_time_kernel.restype = C.c_int
    rt._L.esp_llama_time_kernel.argtypes = [C.c_void_p, C.c_int, C.c_int, C.POINTER(C.c_double)]
    out = C.c_double(0)
    _lib.check(rt._L.esp_llama_time_kernel(rt._h, KERNEL_CLASSES.index(name), iters, C.byref(out)))
    return out.value


def time_kernel_dispatch(rt: LlamaRuntime, name: str, iters: int = 8) -> tuple[float, float]:
    """(back-to-back mean, mean kernel duration from events attached to each launch) in microseconds for one GEMV class
    over all layers (invalidates sequence state)."""
    rt._L.esp_llama_time_kernel_dispatch.restype = C.c_int
    rt._L.esp_llama_time_kernel_dispatch.argtypes = [C.c_void_p, C.c_int, C.c_int, C.POINTER(C.c_double), C.POINTER(C.c_double)]
    b2b, own = C.c_double(0), C.c_double(0)
    _lib.check(rt._L.esp_llama_time_kernel_dispatch(rt._h, KERNEL_CLASSES.index(name), iters, C.byref(b2b), C.byref(own)))
    return b2b.value, own.value


def kernel_times(rt: LlamaRuntime, reset: bool = True) -> dict:
    """{class: {"total_us", "launches", "bytes_per_launch", "mean_us", "gbps"}} from HIP events."""
    n = len(KERNEL_CLASSES)
    tot = np.zeros(n, dtype=np.float64)
    cnt = np.zeros(n, dtype=np.int64)
    byt = np.zeros(n, dtype=np.uint64)
    _lib.check(rt._L.esp_llama_kernel_times(rt._h, _ptr(tot), _ptr(cnt), _ptr(byt), int(reset)))
    out = {}
    for i, name in enumerate(KERNEL_CLASSES):
        mean = tot[i] / cnt[i] if cnt[i] else 0.0
        out[name] = {"total_us": float(tot[i]), "launches": int(cnt[i]), "bytes_per_launch": int(byt[i]),
                     "mean_us": float(mean), "gbps": float(byt[i] / mean / 1e3) if mean > 0 and byt[i] else 0.0}
    return out
