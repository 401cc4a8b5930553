"""Kernel handles and surfaces over the C ABI, in the shape of the reference's ANEKernel
(Sources/ANERuntime/ANEKernel.swift) and SurfaceIO (Sources/ANETypes/SurfaceIO.swift).  The Python
side only marshals pointers; every conversion, copy and kernel runs in the shared library."""
from __future__ import annotations

import ctypes as C

import numpy as np

from . import _lib

COMPILE_ERROR_NONE, COMPILE_ERROR_INVALID_ARGUMENTS, COMPILE_ERROR_DUPLICATE_WEIGHT_PATH = 0, 1, 2
COMPILE_ERROR_SURFACE_ALLOCATION_FAILED, COMPILE_ERROR_COMPILER_FAILURE = 3, 4

_DECLARED = False


def _L() -> C.CDLL:
    global _DECLARED
    L = _lib.load_library()
    if _DECLARED:
        return L
    vp, sz, i32, b, fp, ip = C.c_void_p, C.c_size_t, C.c_int, C.c_bool, C.POINTER(C.c_float), C.POINTER(C.c_int)
    sig = {
        "esp_interop_init": (None, []),
        "esp_interop_create_surface": (vp, [sz]),
        "esp_surface_retain": (vp, [vp]),
        "esp_surface_release": (None, [vp]),
        "esp_surface_bytes": (sz, [vp]),
        "esp_interop_compile": (vp, [vp, sz, C.POINTER(C.c_char_p), C.POINTER(vp), C.POINTER(sz), i32, i32, C.POINTER(sz), i32, C.POINTER(sz)]),
        "esp_interop_eval": (b, [vp]),
        "esp_interop_get_input": (vp, [vp, i32]),
        "esp_interop_get_output": (vp, [vp, i32]),
        "esp_interop_copy_input": (vp, [vp, i32]),
        "esp_interop_copy_output": (vp, [vp, i32]),
        "esp_interop_free": (None, [vp]),
        "esp_interop_compile_count": (i32, []),
        "esp_interop_set_compile_count": (None, [i32]),
        "esp_interop_last_compile_error": (i32, []),
        "esp_interop_set_force_eval_failure": (None, [b]),
        "esp_interop_live_handle_count": (i32, []),
        "esp_interop_last_hw_execution_time_ns": (C.c_uint64, [vp]),
        "esp_interop_has_perf_stats": (b, [vp]),
        "esp_interop_rebind_input": (b, [vp, i32, vp]),
        "esp_interop_cvt_f32_to_f16": (None, [vp, vp, i32]),
        "esp_interop_cvt_f16_to_f32": (None, [vp, vp, i32]),
        "esp_interop_argmax_f16": (None, [vp, i32, ip, fp]),
        "esp_interop_argmax_f16_strided": (None, [vp, i32, i32, ip, fp]),
        "esp_interop_io_copy": (b, [vp, i32, vp, i32, i32, i32]),
        "esp_interop_io_copy_fp16_spatial_slice": (b, [vp, i32, i32, i32, vp, i32, i32, i32, i32]),
        "esp_interop_io_write_fp16_spatial_slice": (b, [vp, i32, i32, i32, vp, i32]),
        "esp_interop_io_read_fp16_spatial_slice": (b, [vp, i32, i32, i32, vp, i32]),
        "esp_interop_io_argmax_fp16_spatial_slice": (b, [vp, i32, i32, i32, i32, ip, fp]),
        "esp_interop_io_write_fp16": (b, [vp, vp, i32, i32]),
        "esp_interop_io_read_fp16": (b, [vp, i32, vp, i32, i32]),
        "esp_interop_io_read_fp16_batched": (b, [vp, i32, C.POINTER(vp), ip, ip, i32]),
        "esp_interop_io_write_fp16_at": (b, [vp, i32, vp, i32, i32]),
        "esp_interop_io_write_embedding_batch_fp16": (b, [vp, i32, i32, vp, i32, i32, vp, i32]),
        "esp_interop_io_argmax_batch_fp16_spatial": (b, [vp, i32, i32, i32, i32, ip, fp]),
        "esp_interop_io_copy_two_fp16_spatial_slices": (b, [vp, i32, i32, i32, vp, i32, i32, i32, vp, i32, i32, i32, vp, i32, i32, i32, i32]),
        "esp_interop_io_argmax_fp16_spatial_slice_with_hint": (b, [vp, i32, i32, i32, i32, vp, i32, i32, ip, fp]),
        "esp_interop_io_write_fp16_at_batched": (b, [vp, ip, C.POINTER(vp), ip, i32, i32]),
        "esp_interop_io_copy_batched": (b, [vp, vp, ip, ip, ip, i32, i32]),
        "esp_interop_io_copy_multi_src": (b, [vp, C.POINTER(vp), ip, ip, ip, i32, i32]),
        "esp_interop_io_argmax_batch_fp16_spatial_parallel": (b, [vp, i32, i32, i32, i32, ip, fp, i32]),
        "esp_interop_io_argmax_batch_fp16_spatial_nolock": (b, [vp, i32, i32, i32, i32, ip, fp, i32]),
        "esp_interop_fused_expansion_argmax_fp16": (b, [vp, i32, i32, i32, i32, vp, i32, i32, ip, fp, i32]),
        "esp_interop_expansion_head_create": (vp, [vp, i32, i32, i32]),
        "esp_interop_expansion_head_argmax": (b, [vp, vp, i32, i32, i32, i32, ip, fp]),
        "esp_interop_expansion_head_free": (None, [vp]),
        "esp_interop_gather_f16_to_f32": (None, [vp, vp, i32, i32]),
        "esp_interop_scatter_f32_to_f16": (None, [vp, vp, i32, i32]),
        "esp_interop_rope_decode": (b, [vp, vp, i32, i32, i32, i32, C.c_float, i32]),
        "esp_interop_kv_cache_scatter": (b, [vp, vp, vp, vp, i32, i32, i32, i32]),
        "esp_interop_decode_sdpa": (b, [vp, vp, vp, vp, i32, i32, i32, i32, i32, i32, i32]),
        "esp_interop_io_lock_write": (b, [vp]),
        "esp_interop_io_unlock_write": (b, [vp]),
        "esp_interop_io_lock_read": (b, [vp]),
        "esp_interop_io_unlock_read": (b, [vp]),
        "esp_interop_io_write_fp16_unlocked": (b, [vp, vp, i32, i32]),
        "esp_interop_io_read_fp16_unlocked": (b, [vp, i32, vp, i32, i32]),
    }
    for name, (res, args) in sig.items():
        fn = getattr(L, name)
        fn.restype, fn.argtypes = res, args
    _DECLARED = True
    return L


def _ptr(a: np.ndarray):
    return a.ctypes.data_as(C.c_void_p)


class SurfaceIOError(RuntimeError):
    """SurfaceIO.swift's argumentOutOfRange / interopCallFailed."""


class Surface:
    """A retained surface: `channels x spatial` fp16 values, channel-first."""

    def __init__(self, ref: int, owned: bool = True):
        self.ref, self._owned = ref, owned

    @classmethod
    def create(cls, nbytes: int) -> "Surface":
        ref = _L().esp_interop_create_surface(nbytes)
        if not ref:
            raise MemoryError("esp_interop_create_surface failed")
        return cls(ref)

    @property
    def bytes(self) -> int:
        return int(_L().esp_surface_bytes(self.ref))

    def release(self) -> None:
        if self._owned and self.ref:
            _L().esp_surface_release(self.ref)
        self.ref = None

    def __del__(self):
        try:
            self.release()
        except Exception:
            pass


def _ok(result: bool, what: str) -> None:
    if not result:
        raise SurfaceIOError(what)


class SurfaceIO:
    """Static helpers with SurfaceIO.swift's names and argument order."""

    @staticmethod
    def writeFP16(to: Surface, data, channels: int, spatial: int) -> None:
        a = np.ascontiguousarray(data, dtype=np.float32)
        _ok(a.size == channels * spatial and _L().esp_interop_io_write_fp16(to.ref, _ptr(a), channels, spatial), "writeFP16")

    @staticmethod
    def writeFP16At(to: Surface, channelOffset: int, data, channels: int, spatial: int) -> None:
        a = np.ascontiguousarray(data, dtype=np.float32)
        _ok(a.size == channels * spatial and _L().esp_interop_io_write_fp16_at(to.ref, channelOffset, _ptr(a), channels, spatial), "writeFP16At")

    @staticmethod
    def readFP16(from_: Surface, channelOffset: int, channels: int, spatial: int) -> np.ndarray:
        out = np.empty(channels * spatial, dtype=np.float32)
        _ok(_L().esp_interop_io_read_fp16(from_.ref, channelOffset, _ptr(out), channels, spatial), "readFP16")
        return out.reshape(channels, spatial)

    @staticmethod
    def readFP16Batched(from_: Surface, spatial: int, regions) -> list[np.ndarray]:
        outs = [np.empty(ch * spatial, dtype=np.float32) for _, ch in regions]
        n = len(regions)
        dst = (C.c_void_p * n)(*[o.ctypes.data for o in outs])
        offs = (C.c_int * n)(*[r[0] for r in regions])
        chs = (C.c_int * n)(*[r[1] for r in regions])
        _ok(_L().esp_interop_io_read_fp16_batched(from_.ref, spatial, dst, offs, chs, n), "readFP16Batched")
        return [o.reshape(ch, spatial) for o, (_, ch) in zip(outs, regions)]

    @staticmethod
    def copyFP16(dst: Surface, dstChannelOffset: int, src: Surface, srcChannelOffset: int, channels: int, spatial: int) -> None:
        _ok(_L().esp_interop_io_copy(dst.ref, dstChannelOffset, src.ref, srcChannelOffset, channels, spatial), "copyFP16")

    @staticmethod
    def copyFP16SpatialSlice(dst: Surface, dstChannelOffset: int, dstSpatialIndex: int, dstSpatial: int, src: Surface,
                             srcChannelOffset: int, srcSpatialIndex: int, srcSpatial: int, channels: int) -> None:
        _ok(_L().esp_interop_io_copy_fp16_spatial_slice(dst.ref, dstChannelOffset, dstSpatialIndex, dstSpatial, src.ref, srcChannelOffset,
                                                        srcSpatialIndex, srcSpatial, channels), "copyFP16SpatialSlice")

    @staticmethod
    def writeFP16SpatialSlice(to: Surface, channelOffset: int, spatialIndex: int, spatial: int, data, channels: int) -> None:
        a = np.ascontiguousarray(data, dtype=np.float32)
        _ok(a.size == channels and _L().esp_interop_io_write_fp16_spatial_slice(to.ref, channelOffset, spatialIndex, spatial, _ptr(a), channels),
            "writeFP16SpatialSlice")

    @staticmethod
    def readFP16SpatialSlice(from_: Surface, channelOffset: int, spatialIndex: int, spatial: int, channels: int) -> np.ndarray:
        out = np.empty(channels, dtype=np.float32)
        _ok(_L().esp_interop_io_read_fp16_spatial_slice(from_.ref, channelOffset, spatialIndex, spatial, _ptr(out), channels), "readFP16SpatialSlice")
        return out

    @staticmethod
    def argmaxFP16SpatialSlice(from_: Surface, channelOffset: int, spatialIndex: int, spatial: int, channels: int) -> tuple[int, float]:
        idx, val = C.c_int(-1), C.c_float(0)
        _ok(_L().esp_interop_io_argmax_fp16_spatial_slice(from_.ref, channelOffset, spatialIndex, spatial, channels, C.byref(idx), C.byref(val)),
            "argmaxFP16SpatialSlice")
        return idx.value, val.value

    @staticmethod
    def writeEmbeddingBatchFP16(to: Surface, channelOffset: int, spatial: int, embeddingTable, vocabSize: int, dim: int, tokenIDs) -> None:
        table = np.ascontiguousarray(embeddingTable, dtype=np.float32)
        ids = np.ascontiguousarray(tokenIDs, dtype=np.uint16)
        _ok(table.size == vocabSize * dim and _L().esp_interop_io_write_embedding_batch_fp16(to.ref, channelOffset, spatial, _ptr(table), vocabSize, dim,
                                                                                               _ptr(ids), ids.size), "writeEmbeddingBatchFP16")

    @staticmethod
    def argmaxBatchFP16Spatial(from_: Surface, channelOffset: int, spatial: int, channels: int, streamCount: int):
        idx = (C.c_int * max(streamCount, 1))()
        val = (C.c_float * max(streamCount, 1))()
        _ok(_L().esp_interop_io_argmax_batch_fp16_spatial(from_.ref, channelOffset, spatial, channels, streamCount, idx, val), "argmaxBatchFP16Spatial")
        return list(idx[:streamCount]), list(val[:streamCount])


    @staticmethod
    def copyTwoFP16SpatialSlices(dst0: Surface, dst0ChannelOffset: int, dst0SpatialIndex: int, dst0Spatial: int, src0: Surface, src0ChannelOffset: int,
                                 src0SpatialIndex: int, src0Spatial: int, dst1: Surface, dst1ChannelOffset: int, dst1SpatialIndex: int, dst1Spatial: int,
                                 src1: Surface, src1ChannelOffset: int, src1SpatialIndex: int, src1Spatial: int, channels: int) -> None:
        """SurfaceIO.swift:285-339."""
        _ok(_L().esp_interop_io_copy_two_fp16_spatial_slices(
            dst0.ref, dst0ChannelOffset, dst0SpatialIndex, dst0Spatial, src0.ref, src0ChannelOffset, src0SpatialIndex, src0Spatial,
            dst1.ref, dst1ChannelOffset, dst1SpatialIndex, dst1Spatial, src1.ref, src1ChannelOffset, src1SpatialIndex, src1Spatial, channels),
            "copyTwoFP16SpatialSlices")

    @staticmethod
    def argmaxFP16SpatialSliceWithHint(from_: Surface, channelOffset: int, spatialIndex: int, spatial: int, channels: int, hint: Surface,
                                       hintSpatialIndex: int, hintSpatial: int) -> tuple[int, float]:
        """SurfaceIO.swift:433-474: the hint surface holds the column's maximum (the classifier kernel's second output)."""
        idx, val = C.c_int(-1), C.c_float(0)
        _ok(_L().esp_interop_io_argmax_fp16_spatial_slice_with_hint(from_.ref, channelOffset, spatialIndex, spatial, channels, hint.ref, hintSpatialIndex,
                                                                   hintSpatial, C.byref(idx), C.byref(val)), "argmaxFP16SpatialSliceWithHint")
        return idx.value, val.value

    @staticmethod
    def writeFP16AtBatched(to: Surface, spatial: int, regions) -> None:
        """regions: (channelOffset, data, channels) triples (SurfaceIO.swift:190-229); all are checked before any is written."""
        keep = [np.ascontiguousarray(d, dtype=np.float32) for _, d, _ in regions]
        n = len(regions)
        offs = (C.c_int * max(n, 1))(*[r[0] for r in regions])
        chans = (C.c_int * max(n, 1))(*[r[2] for r in regions])
        for a, (_, _, ch) in zip(keep, regions):
            if a.size != ch * spatial:
                raise SurfaceIOError("writeFP16AtBatched: data size does not match channels x spatial")
        srcs = (C.c_void_p * max(n, 1))(*[a.ctypes.data for a in keep])
        _ok(_L().esp_interop_io_write_fp16_at_batched(to.ref, offs, srcs, chans, n, spatial), "writeFP16AtBatched")

    @staticmethod
    def copyFP16Batched(dst: Surface, src: Surface, spatial: int, regions) -> None:
        """regions: (dstChannelOffset, srcChannelOffset, channels) triples (SurfaceIO.swift:672-716)."""
        n = len(regions)
        d = (C.c_int * max(n, 1))(*[r[0] for r in regions])
        s = (C.c_int * max(n, 1))(*[r[1] for r in regions])
        c = (C.c_int * max(n, 1))(*[r[2] for r in regions])
        _ok(_L().esp_interop_io_copy_batched(dst.ref, src.ref, d, s, c, n, spatial), "copyFP16Batched")

    @staticmethod
    def copyFP16FromMultipleSources(dst: Surface, spatial: int, regions) -> None:
        """regions: (source, dstChannelOffset, srcChannelOffset, channels) (SurfaceIO.swift:783-828)."""
        n = len(regions)
        srcs = (C.c_void_p * max(n, 1))(*[r[0].ref for r in regions])
        d = (C.c_int * max(n, 1))(*[r[1] for r in regions])
        s = (C.c_int * max(n, 1))(*[r[2] for r in regions])
        c = (C.c_int * max(n, 1))(*[r[3] for r in regions])
        _ok(_L().esp_interop_io_copy_multi_src(dst.ref, srcs, d, s, c, n, spatial), "copyFP16FromMultipleSources")

    @staticmethod
    def _argmax_blocks(fn, what, from_, channelOffset, spatial, channels, streamCount, nBlocks):
        idx = (C.c_int * max(streamCount, 1))()
        val = (C.c_float * max(streamCount, 1))()
        _ok(fn(from_.ref, channelOffset, spatial, channels, streamCount, idx, val, nBlocks), what)
        return list(idx[:streamCount]), list(val[:streamCount])

    @staticmethod
    def argmaxBatchFP16SpatialParallel(from_: Surface, channelOffset: int, spatial: int, channels: int, streamCount: int, nBlocks: int = 4):
        """SurfaceIO.swift:542-578."""
        return SurfaceIO._argmax_blocks(_L().esp_interop_io_argmax_batch_fp16_spatial_parallel, "argmaxBatchFP16SpatialParallel", from_, channelOffset,
                                        spatial, channels, streamCount, nBlocks)

    @staticmethod
    def argmaxBatchFP16SpatialNolock(from_: Surface, channelOffset: int, spatial: int, channels: int, streamCount: int, nBlocks: int = 4):
        """SurfaceIO.swift:580-615."""
        return SurfaceIO._argmax_blocks(_L().esp_interop_io_argmax_batch_fp16_spatial_nolock, "argmaxBatchFP16SpatialNolock", from_, channelOffset,
                                        spatial, channels, streamCount, nBlocks)

    @staticmethod
    def fusedExpansionArgmax(projSurface: Surface, projChannelOffset: int, spatial: int, bottleneck: int, groups: int, expansionWeights, vocabSize: int,
                             streamCount: int, nBlocks: int = 4):
        """SurfaceIO.swift:617-670; expansionWeights: fp16 bits [vocab, bottleneck / groups]."""
        w = np.ascontiguousarray(expansionWeights, dtype=np.uint16)
        if groups <= 0 or bottleneck % groups != 0 or w.size != vocabSize * (bottleneck // groups):
            raise SurfaceIOError("fusedExpansionArgmax: weight count does not match vocab x bottleneck / groups")
        idx = (C.c_int * max(streamCount, 1))()
        val = (C.c_float * max(streamCount, 1))()
        _ok(_L().esp_interop_fused_expansion_argmax_fp16(projSurface.ref, projChannelOffset, spatial, bottleneck, groups, _ptr(w), vocabSize, streamCount,
                                                         idx, val, nBlocks), "fusedExpansionArgmax")
        return list(idx[:streamCount]), list(val[:streamCount])


class FusedExpansionArgmax:
    """MetalExpansionArgmax.swift:966-1088: the factored head's expansion weights resident on the GPU; run() returns one token per lane.
    expansionWeights: fp16 bits [vocab, bottleneck / groups]."""

    def __init__(self, expansionWeights, bottleneck: int, vocabSize: int, spatial: int, groups: int = 1):
        w = np.ascontiguousarray(expansionWeights, dtype=np.uint16)
        if bottleneck <= 0 or vocabSize <= 0 or spatial <= 0:
            raise SurfaceIOError("all dimensions must be > 0")
        if groups <= 0 or bottleneck % groups != 0 or w.size < vocabSize * (bottleneck // groups):
            raise SurfaceIOError("wExpand too small")
        self.bottleneck, self.vocabSize, self.spatial, self.groups = bottleneck, vocabSize, spatial, groups
        self.ref = _L().esp_interop_expansion_head_create(_ptr(w), bottleneck, groups, vocabSize)
        if not self.ref:
            raise SurfaceIOError("FusedExpansionArgmax: " + _lib.last_error())

    def run(self, projectedSurface: Surface, streamCount: int = None, channelOffset: int = 0, fp32Sums: bool = False, withValues: bool = False):
        n = self.spatial if streamCount is None else streamCount
        idx = (C.c_int * max(n, 1))()
        val = (C.c_float * max(n, 1))()
        _ok(_L().esp_interop_expansion_head_argmax(self.ref, projectedSurface.ref, channelOffset, self.spatial, n, 1 if fp32Sums else 0, idx, val),
            "FusedExpansionArgmax.run")
        return (list(idx[:n]), list(val[:n])) if withValues else list(idx[:n])

    def close(self):
        if self.ref:
            _L().esp_interop_expansion_head_free(self.ref)
            self.ref = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


def gather_f16_to_f32(bits, count: int, stride: int) -> np.ndarray:
    a = np.ascontiguousarray(bits, dtype=np.uint16)
    assert count == 0 or (count - 1) * stride < a.size
    out = np.empty(count, dtype=np.float32)
    _L().esp_interop_gather_f16_to_f32(_ptr(out), _ptr(a), count, stride)
    return out


def scatter_f32_to_f16(dst_bits: np.ndarray, values, stride: int) -> None:
    v = np.ascontiguousarray(values, dtype=np.float32)
    assert dst_bits.dtype == np.uint16 and dst_bits.flags.c_contiguous and (v.size == 0 or (v.size - 1) * stride < dst_bits.size)
    _L().esp_interop_scatter_f32_to_f16(_ptr(dst_bits), _ptr(v), v.size, stride)


def rope_decode(q: Surface, k: Surface, nHeads: int, nKVHeads: int, headDim: int, position: int, theta: float, laneSpatial: int) -> None:
    """rope_decode of the hybrid decode path (MetalAttentionKernel.swift:1756-1795) on surfaces resident on the device."""
    if not _L().esp_interop_rope_decode(q.ref, k.ref, nHeads, nKVHeads, headDim, position, theta, laneSpatial):
        raise ANEError("evaluationFailed", "rope_decode: " + _lib.last_error())


def kv_cache_scatter(kSrc: Surface, vSrc: Surface, kCache: Surface, vCache: Surface, kvDim: int, tokenIndex: int, cacheStride: int, laneSpatial: int) -> None:
    """kv_cache_scatter (MetalAttentionKernel.swift:1805-1820)."""
    if not _L().esp_interop_kv_cache_scatter(kSrc.ref, vSrc.ref, kCache.ref, vCache.ref, kvDim, tokenIndex, cacheStride, laneSpatial):
        raise ANEError("evaluationFailed", "kv_cache_scatter: " + _lib.last_error())


def decode_sdpa(q: Surface, kCache: Surface, vCache: Surface, context: Surface, heads: int, kvHeads: int, headDim: int, visibleTokens: int, tokenBase: int,
                cacheStride: int, laneSpatial: int) -> None:
    """fused_decode_sdpa (MetalAttentionKernel.swift:1824-1886)."""
    if not _L().esp_interop_decode_sdpa(q.ref, kCache.ref, vCache.ref, context.ref, heads, kvHeads, headDim, visibleTokens, tokenBase, cacheStride, laneSpatial):
        raise ANEError("evaluationFailed", "decode_sdpa: " + _lib.last_error())


def cvt_f32_to_f16(values) -> np.ndarray:
    a = np.ascontiguousarray(values, dtype=np.float32)
    out = np.empty(a.size, dtype=np.uint16)
    _L().esp_interop_cvt_f32_to_f16(_ptr(out), _ptr(a), a.size)
    return out


def cvt_f16_to_f32(bits) -> np.ndarray:
    a = np.ascontiguousarray(bits, dtype=np.uint16)
    out = np.empty(a.size, dtype=np.float32)
    _L().esp_interop_cvt_f16_to_f32(_ptr(out), _ptr(a), a.size)
    return out


def argmax_f16(bits, stride: int = 1, count: int | None = None) -> tuple[int, float]:
    a = np.ascontiguousarray(bits, dtype=np.uint16)
    n = a.size // stride if count is None else count
    idx, val = C.c_int(-1), C.c_float(0)
    _L().esp_interop_argmax_f16_strided(_ptr(a), n, stride, C.byref(idx), C.byref(val))
    return idx.value, val.value


class ANEError(RuntimeError):
    """ANEKernel.swift's compilationFailed / evaluationFailed / surfaceAllocationFailed / invalidArguments."""

    def __init__(self, kind: str, detail: str = ""):
        super().__init__(f"{kind}: {detail}" if detail else kind)
        self.kind = kind


def program_text(kernel: str, fmt: str, spatial: int = 1, lanes: int = 1, norm_eps: float = 1e-5, **dims) -> str:
    lines = ["program: espresso.hip/1", f"kernel: {kernel}", f"format: {fmt}", f"spatial: {spatial}", f"lanes: {lanes}", f"norm_eps: {norm_eps!r}"]
    lines += [f"{k}: {v}" for k, v in dims.items()]
    return "\n".join(lines) + "\n"


class ANEKernel:
    """One compiled kernel set with its input and output surfaces (ANEKernel.swift:30-136)."""

    def __init__(self, milText: str, weights: list[tuple[str, bytes]], inputSizes: list[int], outputSizes: list[int]):
        L = _L()
        text = milText.encode()
        n = len(weights)
        paths = (C.c_char_p * max(n, 1))(*[w[0].encode() for w in weights])
        keep = [np.frombuffer(bytes(w[1]), dtype=np.uint8) for w in weights]
        datas = (C.c_void_p * max(n, 1))(*[k.ctypes.data for k in keep])
        lens = (C.c_size_t * max(n, 1))(*[k.size for k in keep])
        ins = (C.c_size_t * max(len(inputSizes), 1))(*inputSizes)
        outs = (C.c_size_t * max(len(outputSizes), 1))(*outputSizes)
        buf = np.frombuffer(text, dtype=np.uint8)
        self._h = L.esp_interop_compile(_ptr(buf), buf.size, paths, datas, lens, n, len(inputSizes), ins, len(outputSizes), outs)
        if not self._h:
            code = L.esp_interop_last_compile_error()
            kind = {COMPILE_ERROR_INVALID_ARGUMENTS: "invalidArguments", COMPILE_ERROR_DUPLICATE_WEIGHT_PATH: "invalidArguments",
                    COMPILE_ERROR_SURFACE_ALLOCATION_FAILED: "surfaceAllocationFailed"}.get(code, "compilationFailed")
            raise ANEError(kind, _lib.last_error())

    def eval(self) -> None:
        if not _L().esp_interop_eval(self._h):
            raise ANEError("evaluationFailed", _lib.last_error())

    def inputSurface(self, index: int) -> Surface:
        ref = _L().esp_interop_copy_input(self._h, index)
        if not ref:
            raise ANEError("invalidArguments", f"input index {index}")
        return Surface(ref)

    def outputSurface(self, index: int) -> Surface:
        ref = _L().esp_interop_copy_output(self._h, index)
        if not ref:
            raise ANEError("invalidArguments", f"output index {index}")
        return Surface(ref)

    def rebindInput(self, index: int, surface: Surface) -> None:
        if not _L().esp_interop_rebind_input(self._h, index, surface.ref):
            raise ANEError("invalidArguments", "rebindInput")

    def lastHWExecutionTimeNS(self) -> int:
        return int(_L().esp_interop_last_hw_execution_time_ns(self._h))

    def free(self) -> None:
        if self._h:
            _L().esp_interop_free(self._h)
            self._h = None

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass
