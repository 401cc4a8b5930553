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
