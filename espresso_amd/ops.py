"""numpy-facing wrappers over the C ABI's GGUF-block and GEMV entry points."""
from __future__ import annotations

import ctypes as C

import numpy as np

from . import _lib


def _ptr(a: np.ndarray):
    return a.ctypes.data_as(C.c_void_p)


def init() -> None:
    _lib.check(_lib.load_library().esp_init())


def device_info() -> dict:
    L = _lib.load_library()
    name = C.create_string_buffer(128)
    cus, hbm = C.c_int(0), C.c_size_t(0)
    _lib.check(L.esp_device_info(name, 128, C.byref(cus), C.byref(hbm)))
    return {"name": name.value.decode(), "compute_units": cus.value, "hbm_bytes": hbm.value}


def format_bytes(fmt: int, elements: int) -> int:
    return int(_lib.load_library().esp_format_bytes(fmt, elements))


def dequantize(fmt: int, blocks: np.ndarray, elements: int) -> np.ndarray:
    """DequantDispatcher.dequantize: GGUF-layout blocks -> fp32 (decoded on the GPU)."""
    blocks = np.ascontiguousarray(blocks, dtype=np.uint8)
    out = np.empty(elements, dtype=np.float32)
    _lib.check(_lib.load_library().esp_dequantize(fmt, _ptr(blocks), elements, _ptr(out)))
    return out


class Matrix:
    """A [rows, cols] weight resident in HBM in the GEMV kernels' layout."""

    def __init__(self, fmt: int, blocks: np.ndarray, rows: int, cols: int):
        L = _lib.load_library()
        blocks = np.ascontiguousarray(blocks, dtype=np.uint8)
        expected = L.esp_format_bytes(fmt, rows * cols)
        if expected == 0 or blocks.size != expected:
            raise ValueError(f"{blocks.size} bytes given, format {fmt} needs {expected} for {rows}x{cols}")
        self._h = L.esp_matrix_create(fmt, _ptr(blocks), rows, cols)
        if not self._h:
            raise _lib.EspressoError(-1, _lib.last_error())
        self.format, self.rows, self.cols = fmt, rows, cols

    def close(self) -> None:
        if self._h:
            _lib.load_library().esp_matrix_free(self._h)
            self._h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    @property
    def bytes(self) -> int:
        return int(_lib.load_library().esp_matrix_bytes(self._h))

    @property
    def resident_bytes(self) -> int:
        return int(_lib.load_library().esp_matrix_resident_bytes(self._h))

    def read_tiled(self) -> np.ndarray:
        """The tiled copy the matrix-core GEMVs read, as bytes (empty when the matrix keeps none)."""
        n = self.resident_bytes - self.bytes
        out = np.empty(max(n, 1), dtype=np.uint8)
        got = _lib.load_library().esp_matrix_read_tiled(self._h, _ptr(out), out.size)
        if got < 0:
            _lib.check(int(got))
        return out[:got]

    def dequantize(self) -> np.ndarray:
        out = np.empty(self.rows * self.cols, dtype=np.float32)
        _lib.check(_lib.load_library().esp_matrix_dequantize(self._h, _ptr(out)))
        return out.reshape(self.rows, self.cols)

    def gemv(self, x_f16: np.ndarray, residual: np.ndarray | None = None) -> np.ndarray:
        x = np.ascontiguousarray(x_f16, dtype=np.float16).reshape(-1, self.cols)
        batch = x.shape[0]
        y = np.empty((batch, self.rows), dtype=np.float32)
        res = None
        if residual is not None:
            res = np.ascontiguousarray(residual, dtype=np.float32).reshape(batch, self.rows)
        _lib.check(_lib.load_library().esp_gemv(self._h, _ptr(x), batch, _ptr(y), _ptr(res) if res is not None else None))
        return y

    def matmul_f32(self, x: np.ndarray, residual: np.ndarray | None = None) -> np.ndarray:
        """fp32 activations [rows][cols] against the matrix with no operand rounded (esp_matmul_f32; Q4_K)."""
        x = np.ascontiguousarray(x, dtype=np.float32).reshape(-1, self.cols)
        rows = x.shape[0]
        y = np.empty((rows, self.rows), dtype=np.float32)
        res = None
        if residual is not None:
            res = np.ascontiguousarray(residual, dtype=np.float32).reshape(rows, self.rows)
        _lib.check(_lib.load_library().esp_matmul_f32(self._h, _ptr(x), rows, _ptr(y), _ptr(res) if res is not None else None))
        return y

    def matmul_f32_swiglu(self, x: np.ndarray) -> np.ndarray:
        """SiLU(gate) * up of the exact Q4_K product for a matrix of interleaved gate / up rows (esp_matmul_f32_swiglu; test aid)."""
        x = np.ascontiguousarray(x, dtype=np.float32).reshape(-1, self.cols)
        act = np.empty((x.shape[0], self.rows // 2), dtype=np.float32)
        _lib.check(_lib.load_library().esp_matmul_f32_swiglu(self._h, _ptr(x), x.shape[0], _ptr(act)))
        return act

    def time_gemv(self, batch: int = 1, warmup: int = 10, iters: int = 50, rotate: int = 1) -> dict:
        mean, best = C.c_double(0), C.c_double(0)
        _lib.check(_lib.load_library().esp_gemv_time(self._h, batch, warmup, iters, rotate, C.byref(mean), C.byref(best)))
        return {"mean_us": mean.value, "best_us": best.value}


class Int4Classifier:
    """INT4Classifier over TensorBufferINT4: per-row 4-bit quantisation on the host, logits and argmax on the GPU."""

    def __init__(self, weights: np.ndarray):
        w = np.ascontiguousarray(weights, dtype=np.float32)
        self.rows, self.cols = w.shape
        L = _lib.load_library()
        L.esp_int4_classifier_create.restype = C.c_void_p
        L.esp_int4_classifier_create.argtypes = [C.c_void_p, C.c_int, C.c_int]
        L.esp_int4_classifier_free.argtypes = [C.c_void_p]
        L.esp_int4_classifier_export.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p]
        L.esp_int4_classifier_matvec_argmax.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.POINTER(C.c_int)]
        self._h = L.esp_int4_classifier_create(_ptr(w), self.rows, self.cols)
        if not self._h:
            raise _lib.EspressoError(-1, _lib.last_error())

    def export(self):
        packed = np.empty((self.rows, (self.cols + 1) // 2), np.uint8)
        scales, biases = np.empty(self.rows, np.float32), np.empty(self.rows, np.float32)
        _lib.check(_lib.load_library().esp_int4_classifier_export(self._h, _ptr(packed), _ptr(scales), _ptr(biases)))
        return packed, scales, biases

    def matvec_argmax(self, x):
        x = np.ascontiguousarray(x, dtype=np.float32)
        logits = np.empty(self.rows, np.float32)
        idx = C.c_int(-1)
        _lib.check(_lib.load_library().esp_int4_classifier_matvec_argmax(self._h, _ptr(x), _ptr(logits), C.byref(idx)))
        return logits, idx.value

    def close(self):
        if self._h:
            _lib.load_library().esp_int4_classifier_free(self._h)
            self._h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


def gemv_stamps(m: "Matrix", batch: int = 1, launches: int = 8, capacity: int = 16384) -> tuple[np.ndarray, float]:
    """([wavefronts][4] wall-clock stamps (100 MHz ticks: start, staged, first weights consumed, end), microseconds from
    this launch's first wavefront start to the next launch's) of one Q4_K GEMV launch inside a back-to-back train over
    copies of the matrix that exceed the caches."""
    L = _lib.load_library()
    L.esp_gemv_stamps.restype = C.c_int
    L.esp_gemv_stamps.argtypes = [C.c_void_p, C.c_int, C.c_int, C.c_void_p, C.c_int, C.POINTER(C.c_int), C.POINTER(C.c_double)]
    out = np.zeros((capacity, 4), dtype=np.uint64)
    n, us = C.c_int(0), C.c_double(0)
    _lib.check(L.esp_gemv_stamps(m._h, batch, launches, _ptr(out), capacity, C.byref(n), C.byref(us)))
    return out[:n.value], us.value


def set_tuning(key: str, value: int) -> None:
    """Kernel-selection switch (esp_set_tuning)."""
    L = _lib.load_library()
    L.esp_set_tuning.restype = C.c_int
    L.esp_set_tuning.argtypes = [C.c_char_p, C.c_int]
    _lib.check(L.esp_set_tuning(key.encode(), value))


def hbm_read_probe(nbytes: int = 1 << 30, iters: int = 10) -> float:
    """GB/s a plain streaming-read kernel reaches over `nbytes` of HBM."""
    L = _lib.load_library()
    L.esp_hbm_read_probe.restype = C.c_int
    L.esp_hbm_read_probe.argtypes = [C.c_size_t, C.c_int, C.POINTER(C.c_double)]
    out = C.c_double(0)
    _lib.check(L.esp_hbm_read_probe(nbytes, iters, C.byref(out)))
    return out.value


def hbm_read_probe_pairs(bytes_per_launch: int, pair_bytes: int = 2304, workgroups: int = 512, wavefronts: int = 8, copies: int = 16,
                         launches: int = 64) -> dict:
    """Mean microseconds and GB/s of a reader with a persistent Q4_K GEMV's grid and loads over `bytes_per_launch` per launch
    (defaults: the matrix-core kernel's 512 workgroups of eight wavefronts, one 2304-byte tile ahead per wavefront)."""
    L = _lib.load_library()
    L.esp_hbm_read_probe_pairs.restype = C.c_int
    L.esp_hbm_read_probe_pairs.argtypes = [C.c_size_t, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, C.POINTER(C.c_double), C.POINTER(C.c_double)]
    us, gbps = C.c_double(0), C.c_double(0)
    _lib.check(L.esp_hbm_read_probe_pairs(bytes_per_launch, pair_bytes, workgroups, wavefronts, copies, launches, C.byref(us), C.byref(gbps)))
    return {"mean_us": us.value, "gbps": gbps.value}


def synth_weights(fmt: int, seed: int, std: float, elements: int) -> np.ndarray:
    """Seeded N(0, std) weights quantised on the GPU into GGUF-layout blocks (uint8 array)."""
    L = _lib.load_library()
    out = np.empty(int(L.esp_format_bytes(fmt, elements)), dtype=np.uint8)
    _lib.check(L.esp_synth_weights(fmt, C.c_uint64(seed), C.c_float(std), elements, _ptr(out)))
    return out
