"""ctypes loader for libespresso_hip.so.  No compute happens in Python and nothing here falls back
to a CPU path: if the library is missing it is built with hipcc, and if that fails the import error
is raised to the caller."""
from __future__ import annotations

import ctypes as C
import os

from . import build as _build

_LIB = None

FORMAT_F32, FORMAT_F16, FORMAT_Q4_0, FORMAT_Q8_0, FORMAT_Q4_K = 0, 1, 2, 8, 12
FORMAT_NAMES = {"f32": 0, "f16": 1, "q4_0": 2, "q8_0": 8, "q4_k": 12}


class EspressoError(RuntimeError):
    def __init__(self, code: int, message: str):
        super().__init__(f"[{code}] {message}")
        self.code = code
        self.message = message


def library_path() -> str:
    return _build.LIB_PATH


def load_library() -> C.CDLL:
    global _LIB
    if _LIB is not None:
        return _LIB
    path = library_path()
    if not os.path.exists(path):
        _build.build()
    lib = C.CDLL(path)
    _declare(lib)
    _declare_llama(lib)
    _LIB = lib
    return lib


def check(rc: int) -> None:
    if rc != 0:
        raise EspressoError(rc, load_library().esp_last_error().decode())


def last_error() -> str:
    return load_library().esp_last_error().decode()


def _declare(L: C.CDLL) -> None:
    vp, sz, i32 = C.c_void_p, C.c_size_t, C.c_int
    dp = C.POINTER(C.c_double)
    L.esp_init.restype = i32
    L.esp_last_error.restype = C.c_char_p
    L.esp_device_info.restype = i32
    L.esp_device_info.argtypes = [C.c_char_p, sz, C.POINTER(i32), C.POINTER(sz)]
    L.esp_format_bytes.restype = sz
    L.esp_format_bytes.argtypes = [i32, sz]
    L.esp_dequantize.restype = i32
    L.esp_dequantize.argtypes = [i32, vp, sz, vp]
    L.esp_matrix_create.restype = vp
    L.esp_matrix_create.argtypes = [i32, vp, i32, i32]
    L.esp_matrix_free.argtypes = [vp]
    L.esp_matrix_bytes.restype = sz
    L.esp_matrix_bytes.argtypes = [vp]
    L.esp_matrix_dequantize.restype = i32
    L.esp_matrix_dequantize.argtypes = [vp, vp]
    L.esp_gemv.restype = i32
    L.esp_gemv.argtypes = [vp, vp, i32, vp, vp]
    L.esp_gemv_time.restype = i32
    L.esp_gemv_time.argtypes = [vp, i32, i32, i32, i32, dp, dp]


class LlamaConfigStruct(C.Structure):
    _fields_ = [(n, C.c_int32) for n in ("n_layer", "n_head", "n_kv_head", "d_model", "head_dim", "hidden_dim", "vocab", "max_seq")] + \
               [("norm_eps", C.c_float), ("rope_theta", C.c_float), ("eos_token", C.c_int32), ("kv_format", C.c_int32),
                ("max_sequences", C.c_int32)]


class GenerationStatsStruct(C.Structure):
    _fields_ = [("generated", C.c_int32), ("prefill_ms", C.c_double), ("decode_ms", C.c_double),
                ("first_token_latency_ms", C.c_double), ("tokens_per_second", C.c_double)]


class TwoTokenStatsStruct(C.Structure):
    _fields_ = [(n, C.c_int32) for n in ("passes", "committed_total", "accepted_total", "reference_passes",
                                         "reference_committed_total", "reference_accepted_total")]


def _declare_llama(L: C.CDLL) -> None:
    vp, sz, i32 = C.c_void_p, C.c_size_t, C.c_int
    L.esp_llama_create.restype = vp
    L.esp_llama_create.argtypes = [C.POINTER(LlamaConfigStruct)]
    L.esp_llama_free.argtypes = [vp]
    L.esp_llama_set_weight.restype = i32
    L.esp_llama_set_weight.argtypes = [vp, i32, i32, i32, vp, sz]
    L.esp_llama_finalize.restype = i32
    L.esp_llama_finalize.argtypes = [vp]
    L.esp_llama_weight_bytes.restype = sz
    L.esp_llama_weight_bytes.argtypes = [vp]
    L.esp_llama_reset.restype = i32
    L.esp_llama_reset.argtypes = [vp]
    L.esp_llama_prefill.restype = i32
    L.esp_llama_prefill.argtypes = [vp, i32, vp, i32]
    L.esp_llama_advance.restype = i32
    L.esp_llama_advance.argtypes = [vp, i32, C.c_uint32]
    L.esp_llama_select_greedy_token.restype = i32
    L.esp_llama_select_greedy_token.argtypes = [vp, i32, C.POINTER(C.c_uint32)]
    L.esp_llama_visible_token_count.restype = i32
    L.esp_llama_visible_token_count.argtypes = [vp, i32]
    L.esp_llama_set_visible_token_count.restype = i32
    L.esp_llama_set_visible_token_count.argtypes = [vp, i32, i32]
    L.esp_llama_read_last_hidden.restype = i32
    L.esp_llama_read_last_hidden.argtypes = [vp, i32, vp]
    L.esp_llama_read_logits.restype = i32
    L.esp_llama_read_logits.argtypes = [vp, i32, vp]
    L.esp_llama_generate.restype = i32
    L.esp_llama_generate.argtypes = [vp, vp, i32, i32, vp, C.POINTER(i32), C.POINTER(GenerationStatsStruct), vp]
    L.esp_llama_generate_two_token.restype = i32
    L.esp_llama_generate_two_token.argtypes = [vp, vp, vp, i32, i32, i32, vp, C.POINTER(i32),
                                               C.POINTER(GenerationStatsStruct), C.POINTER(TwoTokenStatsStruct)]
    L.esp_llama_continue_greedy.restype = i32
    L.esp_llama_continue_greedy.argtypes = [vp, i32, i32, vp]
    L.esp_llama_set_kernel_timing.restype = i32
    L.esp_llama_set_kernel_timing.argtypes = [vp, i32]
    L.esp_llama_kernel_times.restype = i32
    L.esp_llama_kernel_times.argtypes = [vp, vp, vp, vp, i32]
    L.esp_synth_weights.restype = i32
    L.esp_synth_weights.argtypes = [i32, C.c_uint64, C.c_float, sz, vp]
    L.esp_llama_set_graph_replay.restype = i32
    L.esp_llama_set_graph_replay.argtypes = [vp, i32]
    L.esp_llama_set_merged_attention.restype = i32
    L.esp_llama_set_merged_attention.argtypes = [vp, i32]
    L.esp_matrix_resident_bytes.restype = C.c_size_t
    L.esp_matrix_read_tiled.restype = C.c_longlong
    L.esp_matrix_read_tiled.argtypes = [vp, vp, C.c_size_t]
    L.esp_matrix_resident_bytes.argtypes = [vp]
    L.esp_llama_resident_weight_bytes.restype = C.c_size_t
    L.esp_llama_resident_weight_bytes.argtypes = [vp]
    L.esp_matmul_f32.restype = i32
    L.esp_matmul_f32.argtypes = [vp, vp, i32, vp, vp]
    L.esp_matmul_f32_swiglu.restype = i32
    L.esp_matmul_f32_swiglu.argtypes = [vp, vp, i32, vp]
    L.esp_llama_set_split_activations.restype = i32
    L.esp_llama_set_split_activations.argtypes = [vp, i32]
    L.esp_llama_set_matrix_prefill.restype = i32
    L.esp_llama_set_matrix_prefill.argtypes = [vp, i32]
