"""ctypes binding of the CPU oracle (oracle/liboracle.so).

TEST INFRASTRUCTURE ONLY: imported by tests/, by __graft_entry__.smoke() and by
the cpu_baseline leg of bench.py.  The shipped package never imports it.
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess
from dataclasses import dataclass

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "liboracle.so")

FMT_F32, FMT_F16, FMT_Q4_0, FMT_Q8_0, FMT_Q4_K = 0, 1, 2, 8, 12

W_TOKEN_EMBEDDING, W_FINAL_NORM, W_LM_HEAD = 0, 1, 2
W_RMS_ATT, W_WQ, W_WK, W_WV, W_WO, W_RMS_FFN, W_W1, W_W2, W_W3, W_Q_NORM, W_K_NORM = range(10, 21)


def build() -> str:
    """Compile liboracle.so with gcc (always recompiles)."""
    subprocess.run(["make", "-C", _HERE, "-B", "liboracle.so"], check=True, capture_output=True)
    return _LIB_PATH


class _Config(C.Structure):
    _fields_ = [(n, C.c_int) for n in
                ("n_layer", "n_head", "n_kv_head", "d_model", "head_dim", "hidden_dim", "vocab", "max_seq")] + \
               [("norm_eps", C.c_float), ("rope_theta", C.c_float), ("eos_token", C.c_int),
                ("round_intermediates_fp16", C.c_int), ("gemv_inputs_fp16", C.c_int), ("kv_fp16", C.c_int)]


class _Stats(C.Structure):
    _fields_ = [("passes", C.c_int), ("committed_total", C.c_int), ("accepted_total", C.c_int)]


_lib = None


def lib():
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(_LIB_PATH):
        build()
    L = C.CDLL(_LIB_PATH)
    f32p, u8p, u32p, vp = C.POINTER(C.c_float), C.POINTER(C.c_uint8), C.POINTER(C.c_uint32), C.c_void_p
    L.orc_f32_to_f16.restype = C.c_uint16; L.orc_f32_to_f16.argtypes = [C.c_float]
    L.orc_f16_to_f32.restype = C.c_float; L.orc_f16_to_f32.argtypes = [C.c_uint16]
    L.orc_round_f16_vector.argtypes = [vp, C.c_size_t]
    L.orc_format_bytes.restype = C.c_size_t; L.orc_format_bytes.argtypes = [C.c_int, C.c_size_t]
    L.orc_dequantize.restype = C.c_int; L.orc_dequantize.argtypes = [C.c_int, vp, C.c_size_t, vp]
    L.orc_quantize.restype = C.c_int; L.orc_quantize.argtypes = [C.c_int, vp, C.c_size_t, vp]
    L.orc_q4_k_scale_min.argtypes = [C.c_int, vp, u8p, u8p]
    L.orc_rmsnorm.argtypes = [vp, vp, C.c_float, C.c_int, vp]
    L.orc_per_head_rmsnorm.argtypes = [vp, vp, C.c_int, C.c_int, C.c_float]
    L.orc_matvec.argtypes = [vp, C.c_int, C.c_int, vp, vp]
    L.orc_rope_half_split.argtypes = [vp, C.c_int, C.c_int, C.c_int, C.c_float]
    L.orc_attention_decode.argtypes = [vp, vp, vp, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, vp]
    L.orc_silu_tanh.restype = C.c_float; L.orc_silu_tanh.argtypes = [C.c_float]
    L.orc_partitioned_argmax.restype = C.c_int
    L.orc_partitioned_argmax.argtypes = [vp, vp, C.c_int, C.c_int, C.c_int, C.POINTER(C.c_int)]
    L.orc_naive_argmax.restype = C.c_int; L.orc_naive_argmax.argtypes = [vp, C.c_int]
    L.orc_blob_bytes.restype = C.c_size_t; L.orc_blob_bytes.argtypes = [C.c_size_t]
    L.orc_blob_build.argtypes = [vp, C.c_size_t, vp]
    L.orc_blob_parse.restype = C.c_long; L.orc_blob_parse.argtypes = [vp, C.c_size_t, vp, C.c_size_t]
    L.orc_llama_create.restype = vp; L.orc_llama_create.argtypes = [C.POINTER(_Config)]
    L.orc_llama_free.argtypes = [vp]
    L.orc_llama_set_weight.restype = C.c_int
    L.orc_llama_set_weight.argtypes = [vp, C.c_int, C.c_int, vp, C.c_size_t]
    L.orc_llama_set_weight_blocks.restype = C.c_int
    L.orc_llama_set_weight_blocks.argtypes = [vp, C.c_int, C.c_int, C.c_int, vp, C.c_size_t]
    L.orc_set_threads.argtypes = [C.c_int]
    L.orc_get_threads.restype = C.c_int
    L.orc_llama_reset.argtypes = [vp]
    L.orc_llama_prefill.restype = C.c_int; L.orc_llama_prefill.argtypes = [vp, vp, C.c_int]
    L.orc_llama_advance.restype = C.c_int; L.orc_llama_advance.argtypes = [vp, C.c_uint32]
    L.orc_llama_select_greedy.restype = C.c_uint32; L.orc_llama_select_greedy.argtypes = [vp]
    L.orc_llama_visible.restype = C.c_int; L.orc_llama_visible.argtypes = [vp]
    L.orc_llama_set_visible.argtypes = [vp, C.c_int]
    L.orc_llama_last_hidden.restype = f32p; L.orc_llama_last_hidden.argtypes = [vp]
    L.orc_llama_logits.argtypes = [vp, vp]
    L.orc_llama_top2_margin.restype = C.c_float; L.orc_llama_top2_margin.argtypes = [vp]
    L.orc_llama_capture.restype = vp; L.orc_llama_capture.argtypes = [vp]
    L.orc_llama_rollback.argtypes = [vp, vp]
    L.orc_llama_checkpoint_free.argtypes = [vp]
    L.orc_llama_generate.restype = C.c_int
    L.orc_llama_generate.argtypes = [vp, vp, C.c_int, C.c_int, vp, f32p]
    L.orc_llama_generate_two_token.restype = C.c_int
    L.orc_llama_generate_two_token.argtypes = [vp, vp, vp, C.c_int, C.c_int, vp, C.POINTER(_Stats)]
    _lib = L
    return L


def _f32(a):
    return np.ascontiguousarray(a, dtype=np.float32)


def _ptr(a):
    return a.ctypes.data_as(C.c_void_p)


# ---- fp16 ---------------------------------------------------------------
def f32_to_f16_bits(x: float) -> int:
    return int(lib().orc_f32_to_f16(C.c_float(x)))


def f16_bits_to_f32(bits: int) -> float:
    return float(lib().orc_f16_to_f32(C.c_uint16(bits)))


def round_f16(a):
    out = _f32(a).copy()
    lib().orc_round_f16_vector(_ptr(out), out.size)
    return out


# ---- GGUF blocks ---------------------------------------------------------
def format_bytes(fmt: int, elements: int) -> int:
    return int(lib().orc_format_bytes(fmt, elements))


def quantize(fmt: int, x) -> np.ndarray:
    x = _f32(x).ravel()
    out = np.zeros(format_bytes(fmt, x.size), dtype=np.uint8)
    if lib().orc_quantize(fmt, _ptr(x), x.size, _ptr(out)) != 0:
        raise ValueError(f"unknown format {fmt}")
    return out


def dequantize(fmt: int, blocks, elements: int) -> np.ndarray:
    blocks = np.ascontiguousarray(blocks, dtype=np.uint8)
    assert blocks.size == format_bytes(fmt, elements)
    out = np.empty(elements, dtype=np.float32)
    if lib().orc_dequantize(fmt, _ptr(blocks), elements, _ptr(out)) != 0:
        raise ValueError(f"unknown format {fmt}")
    return out


def q4_k_scale_min(j: int, scales12) -> tuple[int, int]:
    s = np.ascontiguousarray(scales12, dtype=np.uint8)
    sc, m = C.c_uint8(), C.c_uint8()
    lib().orc_q4_k_scale_min(j, _ptr(s), C.byref(sc), C.byref(m))
    return sc.value, m.value


# ---- math helpers --------------------------------------------------------
def rmsnorm(x, w, eps):
    x, w = _f32(x), _f32(w)
    out = np.empty_like(x)
    lib().orc_rmsnorm(_ptr(x), _ptr(w), C.c_float(eps), x.size, _ptr(out))
    return out


def per_head_rmsnorm(values, weights, heads, head_dim, eps):
    v = _f32(values).copy()
    w = _f32(weights)
    lib().orc_per_head_rmsnorm(_ptr(v), _ptr(w), heads, head_dim, C.c_float(eps))
    return v


def set_threads(n: int) -> None:
    """Threads for matvec on large matrices (rows are independent: results are bit-identical for every count)."""
    lib().orc_set_threads(int(n))


def get_threads() -> int:
    return int(lib().orc_get_threads())


def matvec(W, x):
    W, x = _f32(W), _f32(x)
    rows, cols = W.shape
    y = np.empty(rows, dtype=np.float32)
    lib().orc_matvec(_ptr(W), rows, cols, _ptr(x), _ptr(y))
    return y


def rope_half_split(values, heads, head_dim, position, theta=10000.0):
    v = _f32(values).copy()
    lib().orc_rope_half_split(_ptr(v), heads, head_dim, position, C.c_float(theta))
    return v


def attention_decode(q, k_cache, v_cache, heads, kv_heads, head_dim, visible, cache_stride):
    q, k, v = _f32(q), _f32(k_cache), _f32(v_cache)
    out = np.empty(heads * head_dim, dtype=np.float32)
    lib().orc_attention_decode(_ptr(q), _ptr(k), _ptr(v), heads, kv_heads, head_dim, visible, cache_stride, _ptr(out))
    return out


def silu_tanh(x: float) -> float:
    return float(lib().orc_silu_tanh(C.c_float(x)))


def partitioned_argmax(classifier, x, block_size=4000):
    Wm, x = _f32(classifier), _f32(x)
    vocab, dim = Wm.shape
    pruned = C.c_int(0)
    idx = lib().orc_partitioned_argmax(_ptr(Wm), _ptr(x), vocab, dim, block_size, C.byref(pruned))
    return int(idx), int(pruned.value)


def sample_token(logits, temperature: float, unit: float) -> int:
    x = _f32(logits)
    L = lib()
    L.orc_sample_token.restype = C.c_int
    L.orc_sample_token.argtypes = [C.c_void_p, C.c_int, C.c_float, C.c_double]
    return int(L.orc_sample_token(_ptr(x), x.size, temperature, unit))


# ---- INT4 classifier -----------------------------------------------------
def int4_quantize(weights):
    """TensorBufferINT4(quantizing:): (packed [rows][(cols+1)//2] uint8, scales [rows], biases [rows])."""
    w = _f32(weights)
    rows, cols = w.shape
    packed = np.zeros((rows, (cols + 1) // 2), dtype=np.uint8)
    scales, biases = np.empty(rows, np.float32), np.empty(rows, np.float32)
    L = lib()
    L.orc_int4_quantize.restype = None
    L.orc_int4_quantize(_ptr(w), rows, cols, _ptr(packed), _ptr(scales), _ptr(biases))
    return packed, scales, biases


def int4_matvec(packed, scales, biases, x, dim):
    packed, x = np.ascontiguousarray(packed, np.uint8), _f32(x)
    out = np.empty(packed.shape[0], np.float32)
    L = lib()
    L.orc_int4_matvec.restype = None
    L.orc_int4_matvec(_ptr(packed), _ptr(_f32(scales)), _ptr(_f32(biases)), _ptr(x), packed.shape[0], dim, _ptr(out))
    return out


def int4_argmax(packed, scales, biases, x, dim) -> int:
    packed, x = np.ascontiguousarray(packed, np.uint8), _f32(x)
    L = lib()
    L.orc_int4_argmax.restype = C.c_int
    return int(L.orc_int4_argmax(_ptr(packed), _ptr(_f32(scales)), _ptr(_f32(biases)), _ptr(x), packed.shape[0], dim))


# ---- BLOBFILE -----------------------------------------------------------
def blob_build(weights) -> bytes:
    w = _f32(weights).ravel()
    out = np.zeros(int(lib().orc_blob_bytes(w.size)), dtype=np.uint8)
    lib().orc_blob_build(_ptr(w), w.size, _ptr(out))
    return out.tobytes()


def blob_parse(data: bytes):
    buf = np.frombuffer(data, dtype=np.uint8)
    n = lib().orc_blob_parse(_ptr(buf), buf.size, None, 0)
    if n < 0:
        return int(n), None
    out = np.empty(n, dtype=np.float32)
    lib().orc_blob_parse(_ptr(buf), buf.size, _ptr(out), n)
    return int(n), out


# ---- runtime ------------------------------------------------------------
@dataclass
class LlamaConfig:
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
    round_intermediates_fp16: bool = False
    gemv_inputs_fp16: bool = False
    kv_fp16: bool = False


class LlamaRuntime:
    """CPUExactLlamaRuntime restated (RealModelInferenceEngine.swift:548-850)."""

    def __init__(self, cfg: LlamaConfig):
        self.cfg = cfg
        c = _Config(cfg.n_layer, cfg.n_head, cfg.n_kv_head, cfg.d_model, cfg.head_dim, cfg.hidden_dim,
                    cfg.vocab, cfg.max_seq, cfg.norm_eps, cfg.rope_theta, cfg.eos_token,
                    int(cfg.round_intermediates_fp16), int(cfg.gemv_inputs_fp16), int(cfg.kv_fp16))
        self._h = lib().orc_llama_create(C.byref(c))
        if not self._h:
            raise ValueError("invalid config")

    def close(self):
        if self._h:
            lib().orc_llama_free(self._h)
            self._h = None

    def __del__(self):
        self.close()

    def set_weight(self, layer: int, slot: int, data):
        a = _f32(data).ravel()
        rc = lib().orc_llama_set_weight(self._h, layer, slot, _ptr(a), a.size)
        if rc != 0:
            raise ValueError(f"set_weight(layer={layer}, slot={slot}) failed: {rc}")

    def set_weight_blocks(self, layer: int, slot: int, fmt: int, blocks, elements: int):
        """A matrix slot from GGUF blocks, dequantised inside the oracle (no fp32 copy on the Python side)."""
        b = np.ascontiguousarray(blocks, dtype=np.uint8)
        assert b.size == format_bytes(fmt, elements)
        rc = lib().orc_llama_set_weight_blocks(self._h, layer, slot, fmt, _ptr(b), elements)
        if rc != 0:
            raise ValueError(f"set_weight_blocks(layer={layer}, slot={slot}) failed: {rc}")

    def set_gemv_inputs_fp16(self, enabled: bool):
        """Switch the activation mode in place (the weights stay loaded): False, True, or a mask of the inputs that are
        rounded to fp16 (2 attention norm, 4 attention context, 8 FFN norm, 16 SiLU(gate)*up, 32 final norm)."""
        lib().orc_llama_set_gemv_inputs_fp16.argtypes = [C.c_void_p, C.c_int]
        lib().orc_llama_set_gemv_inputs_fp16(self._h, int(enabled))
        self.cfg.gemv_inputs_fp16 = enabled

    def reset(self):
        lib().orc_llama_reset(self._h)

    def prefill(self, tokens) -> int:
        t = np.ascontiguousarray(tokens, dtype=np.uint32)
        return int(lib().orc_llama_prefill(self._h, _ptr(t), t.size))

    def advance(self, token: int) -> int:
        return int(lib().orc_llama_advance(self._h, C.c_uint32(token)))

    def select_greedy(self) -> int:
        return int(lib().orc_llama_select_greedy(self._h))

    @property
    def visible(self) -> int:
        return int(lib().orc_llama_visible(self._h))

    def set_visible(self, n: int):
        lib().orc_llama_set_visible(self._h, n)

    def last_hidden(self) -> np.ndarray:
        p = lib().orc_llama_last_hidden(self._h)
        return np.ctypeslib.as_array(p, shape=(self.cfg.d_model,)).copy()

    def logits(self) -> np.ndarray:
        out = np.empty(self.cfg.vocab, dtype=np.float32)
        lib().orc_llama_logits(self._h, _ptr(out))
        return out

    def top2_margin(self) -> float:
        return float(lib().orc_llama_top2_margin(self._h))

    def capture(self):
        return lib().orc_llama_capture(self._h)

    def rollback(self, ck):
        lib().orc_llama_rollback(self._h, ck)

    @staticmethod
    def free_checkpoint(ck):
        lib().orc_llama_checkpoint_free(ck)

    def generate(self, prompt, max_tokens: int, with_margin: bool = False):
        p = np.ascontiguousarray(prompt, dtype=np.uint32)
        out = np.zeros(max(max_tokens, 1), dtype=np.uint32)
        margin = C.c_float(0)
        n = lib().orc_llama_generate(self._h, _ptr(p), p.size, max_tokens, _ptr(out),
                                     C.byref(margin) if with_margin else None)
        if n < 0:
            raise RuntimeError(f"oracle generate failed: {n}")
        toks = out[:n].tolist()
        return (toks, float(margin.value)) if with_margin else toks


def generate_two_token(full: LlamaRuntime, draft: LlamaRuntime, prompt, max_tokens: int):
    p = np.ascontiguousarray(prompt, dtype=np.uint32)
    out = np.zeros(max(max_tokens, 1), dtype=np.uint32)
    st = _Stats()
    n = lib().orc_llama_generate_two_token(full._h, draft._h, _ptr(p), p.size, max_tokens, _ptr(out), C.byref(st))
    if n < 0:
        raise RuntimeError(f"oracle two-token generate failed: {n}")
    return out[:n].tolist(), {"passes": st.passes, "committed_total": st.committed_total,
                              "accepted_total": st.accepted_total}


def runtime_from_packed(cfg, packed, fmt, n_layer, kv_fp16, max_seq, gemv_inputs_fp16=True):
    """An oracle runtime over a model given as GGUF blocks (the dict espresso_amd.synthetic.build_runtime(keep_packed=True) returns:
    embedding fp16, lm_head and per-layer wq..w3 in `fmt`; norm weights one), dequantised inside the oracle.  `cfg` carries the
    shape (n_head, n_kv_head, d_model, head_dim, hidden_dim, vocab, norm_eps, rope_theta and the derived attention_dim, kv_dim)."""
    ocfg = LlamaConfig(n_layer=n_layer, n_head=cfg.n_head, n_kv_head=cfg.n_kv_head, d_model=cfg.d_model, head_dim=cfg.head_dim,
                       hidden_dim=cfg.hidden_dim, vocab=cfg.vocab, max_seq=max_seq, norm_eps=cfg.norm_eps, rope_theta=cfg.rope_theta,
                       gemv_inputs_fp16=gemv_inputs_fp16, kv_fp16=kv_fp16)
    shapes = {"wq": (cfg.attention_dim, cfg.d_model), "wk": (cfg.kv_dim, cfg.d_model), "wv": (cfg.kv_dim, cfg.d_model),
              "wo": (cfg.d_model, cfg.attention_dim), "w1": (cfg.hidden_dim, cfg.d_model), "w3": (cfg.hidden_dim, cfg.d_model),
              "w2": (cfg.d_model, cfg.hidden_dim)}
    slot = {"wq": W_WQ, "wk": W_WK, "wv": W_WV, "wo": W_WO, "w1": W_W1, "w2": W_W2, "w3": W_W3}
    rt = LlamaRuntime(ocfg)
    n = cfg.vocab * cfg.d_model
    rt.set_weight_blocks(0, W_TOKEN_EMBEDDING, FMT_F16, packed["embedding"], n)
    rt.set_weight(0, W_FINAL_NORM, np.ones(cfg.d_model, np.float32))
    rt.set_weight_blocks(0, W_LM_HEAD, fmt, packed["lm_head"], n)
    for l in range(n_layer):
        rt.set_weight(l, W_RMS_ATT, np.ones(cfg.d_model, np.float32))
        rt.set_weight(l, W_RMS_FFN, np.ones(cfg.d_model, np.float32))
        for k, sl in slot.items():
            r, c = shapes[k]
            rt.set_weight_blocks(l, sl, fmt, packed["layers"][l][k], r * c)
    return rt
