"""Host-side contracts of the kernel-handle / surface API, following the reference's own interop tests
(Tests/ANEInteropTests/ANEInteropTests.swift).  No kernel runs here: surfaces keep a host shadow, and
`compile` validates its pointer contracts before it looks for a device."""
import ctypes as C

import numpy as np
import pytest

import espresso_amd.interop as io
from espresso_amd.interop import Surface, SurfaceIO
from oracle import oracle as orc


def test_init_idempotent_and_nil_handle_accessors():
    L = io._L()
    L.esp_interop_init()
    L.esp_interop_init()                          # ANEInteropTests.swift:285
    assert L.esp_interop_get_input(None, 0) is None and L.esp_interop_get_output(None, 0) is None   # :306
    assert not L.esp_interop_eval(None)
    L.esp_interop_free(None)


def test_create_surface_valid():                  # ANEInteropTests.swift:297
    s = Surface.create(4096)
    assert s.bytes >= 4096
    assert np.all(SurfaceIO.readFP16(s, 0, 64, 32) == 0)


def test_compile_count_set_get_roundtrip():       # ANEInteropTests.swift:311
    L = io._L()
    old = L.esp_interop_compile_count()
    L.esp_interop_set_compile_count(41)
    assert L.esp_interop_compile_count() == 41
    L.esp_interop_set_compile_count(old)


def _compile_raw(paths, datas, lens, n, in_sizes, out_sizes, text=b"program: espresso.hip/1\nkernel: gemv\n"):
    L = io._L()
    buf = np.frombuffer(text, dtype=np.uint8)
    return L.esp_interop_compile(buf.ctypes.data_as(C.c_void_p), buf.size, paths, datas, lens, n,
                                 1, in_sizes, 1, out_sizes)


def test_compile_rejects_invalid_pointer_contracts():   # ANEInteropTests.swift:321
    L = io._L()
    one = (C.c_size_t * 1)(64)
    assert _compile_raw(None, None, None, 1, one, one) is None
    assert L.esp_interop_last_compile_error() == io.COMPILE_ERROR_INVALID_ARGUMENTS
    payload = np.zeros(8, np.uint8)
    paths = (C.c_char_p * 1)(b"@model_path/weights/weight.bin")
    datas = (C.c_void_p * 1)(payload.ctypes.data)
    lens = (C.c_size_t * 1)(8)
    assert _compile_raw(paths, datas, lens, 1, None, one) is None
    assert L.esp_interop_last_compile_error() == io.COMPILE_ERROR_INVALID_ARGUMENTS


def test_compile_rejects_duplicate_weight_paths_and_traversal():   # ANEInteropTests.swift:371, :419
    L = io._L()
    before = L.esp_interop_compile_count()
    one = (C.c_size_t * 1)(64)
    payload = np.zeros(8, np.uint8)
    paths = (C.c_char_p * 2)(b"@model_path/weights/w.bin", b"@model_path/weights/w.bin")
    datas = (C.c_void_p * 2)(payload.ctypes.data, payload.ctypes.data)
    lens = (C.c_size_t * 2)(8, 8)
    assert _compile_raw(paths, datas, lens, 2, one, one) is None
    assert L.esp_interop_last_compile_error() == io.COMPILE_ERROR_DUPLICATE_WEIGHT_PATH
    paths = (C.c_char_p * 1)(b"@model_path/../../escape.bin")
    assert _compile_raw(paths, datas, lens, 1, one, one) is None
    assert L.esp_interop_last_compile_error() == io.COMPILE_ERROR_INVALID_ARGUMENTS
    assert L.esp_interop_compile_count() == before       # :488 failures do not count
    assert L.esp_interop_live_handle_count() == 0


def test_argmax_f16_returns_first_max_index():    # ANEInteropTests.swift:199
    values = [-3, 1, 2, 7, 9, 9, 4, 5, 8, 6, 10, 11, 12, 13, 14, 15, 99, 42, 99, 3, 2, 1, 0, -1]
    idx, val = io.argmax_f16(io.cvt_f32_to_f16(values))
    assert idx == 16 and val == 99.0
    idx, val = io.argmax_f16(io.cvt_f32_to_f16(values), stride=2)    # 9 values at even offsets ... 99 at 16 -> index 8
    assert idx == 8 and val == 99.0


def test_f32_f16_roundtrip_matches_oracle_rounding():    # ANEInteropTests.swift:774
    rng = np.random.default_rng(5)
    x = np.concatenate([rng.normal(0, 1, 4096), rng.normal(0, 1e-6, 512), [0.0, -0.0, 65504.0, 65520.0, 1e-8, 6.1e-5, 1 + 2 ** -11, 1 + 3 * 2 ** -11]]).astype(np.float32)
    bits = io.cvt_f32_to_f16(x)
    want = np.array([orc.f32_to_f16_bits(float(v)) for v in x], dtype=np.uint16)
    assert np.array_equal(bits, want)
    assert np.array_equal(bits, x.astype(np.float16).view(np.uint16))
    back = io.cvt_f16_to_f32(bits)
    assert np.array_equal(back.view(np.uint32), bits.view(np.float16).astype(np.float32).view(np.uint32))


def test_io_copy_between_surfaces():              # ANEInteropTests.swift:796
    channels, spatial = 8, 4
    src, dst = Surface.create(channels * spatial * 2), Surface.create(channels * spatial * 2)
    data = (np.arange(channels * spatial, dtype=np.float32) * 0.25 - 1.0)
    SurfaceIO.writeFP16(src, data, channels, spatial)
    SurfaceIO.copyFP16(dst, 2, src, 0, 6, spatial)
    got = SurfaceIO.readFP16(dst, 0, channels, spatial)
    assert np.all(got[:2] == 0)
    assert np.array_equal(got[2:], data.reshape(channels, spatial)[:6])


def test_io_write_fp16_at_offset_and_batched_read():    # ANEInteropTests.swift:849, SurfaceIO.swift:126
    channels, spatial = 8, 4
    s = Surface.create(channels * spatial * 2)
    part = np.arange(3 * spatial, dtype=np.float32) + 0.5
    SurfaceIO.writeFP16At(s, 4, part, 3, spatial)
    got = SurfaceIO.readFP16(s, 0, channels, spatial)
    assert np.all(got[:4] == 0) and np.all(got[7:] == 0)
    assert np.array_equal(got[4:7].ravel(), part)
    a, b = SurfaceIO.readFP16Batched(s, spatial, [(4, 2), (6, 2)])
    assert np.array_equal(a, got[4:6]) and np.array_equal(b, got[6:8])


def test_io_rejects_invalid_ranges():             # ANEInteropTests.swift:890, :905
    channels, spatial = 8, 4
    a, b = Surface.create(channels * spatial * 2), Surface.create(channels * spatial * 2)
    L = io._L()
    assert not L.esp_interop_io_copy(a.ref, 4, b.ref, 0, 6, spatial)
    assert not L.esp_interop_io_copy(a.ref, -1, b.ref, 0, 2, spatial)
    assert not L.esp_interop_io_copy(a.ref, 0, b.ref, 7, 2, spatial)
    assert not L.esp_interop_io_copy(None, 0, b.ref, 0, 2, spatial)
    x = np.zeros(64, np.float32)
    assert not L.esp_interop_io_write_fp16_at(a.ref, 7, x.ctypes.data_as(C.c_void_p), 2, spatial)
    assert not L.esp_interop_io_write_fp16_at(a.ref, 0, None, 2, spatial)
    assert not L.esp_interop_io_read_fp16(a.ref, 8, x.ctypes.data_as(C.c_void_p), 1, spatial)
    with pytest.raises(io.SurfaceIOError):
        SurfaceIO.readFP16SpatialSlice(a, 0, spatial, spatial, channels)
    with pytest.raises(io.SurfaceIOError):
        SurfaceIO.writeFP16SpatialSlice(a, 0, -1, spatial, np.zeros(channels), channels)


def test_io_copy_same_surface_overlap_uses_memmove_semantics():   # ANEInteropTests.swift:1134
    s = Surface.create(16)
    SurfaceIO.writeFP16(s, np.arange(8, dtype=np.float32), 8, 1)
    SurfaceIO.copyFP16(s, 1, s, 0, 7, 1)
    assert SurfaceIO.readFP16(s, 0, 8, 1).ravel().tolist() == [0, 0, 1, 2, 3, 4, 5, 6]


def test_spatial_slice_write_read_copy_argmax():  # SurfaceIO.swift:251-431
    channels, spatial = 40, 8
    rng = np.random.default_rng(9)
    s, t = Surface.create(channels * spatial * 2), Surface.create(channels * 16 * 2)
    full = rng.normal(0, 1, (channels, spatial)).astype(np.float32)
    SurfaceIO.writeFP16(s, full, channels, spatial)
    col = rng.normal(0, 1, channels).astype(np.float32)
    col[[7, 21]] = 5.0                            # tie: lowest channel wins
    SurfaceIO.writeFP16SpatialSlice(s, 0, 3, spatial, col, channels)
    want = full.astype(np.float16).astype(np.float32)
    want[:, 3] = col.astype(np.float16).astype(np.float32)
    assert np.array_equal(SurfaceIO.readFP16(s, 0, channels, spatial), want)
    assert np.array_equal(SurfaceIO.readFP16SpatialSlice(s, 5, 3, spatial, 10), want[5:15, 3])
    assert SurfaceIO.argmaxFP16SpatialSlice(s, 0, 3, spatial, channels) == (7, 5.0)
    assert SurfaceIO.argmaxFP16SpatialSlice(s, 8, 3, spatial, channels - 8) == (13, 5.0)
    SurfaceIO.copyFP16SpatialSlice(t, 0, 11, 16, s, 0, 3, spatial, channels)
    assert np.array_equal(SurfaceIO.readFP16SpatialSlice(t, 0, 11, 16, channels), want[:, 3])
    assert np.all(SurfaceIO.readFP16SpatialSlice(t, 0, 10, 16, channels) == 0)


def test_embedding_batch_write_and_batch_argmax():   # SurfaceIO.swift:476-540
    vocab, dim, spatial = 50, 12, 8
    rng = np.random.default_rng(11)
    table = rng.normal(0, 1, (vocab, dim)).astype(np.float32)
    s = Surface.create(dim * spatial * 2)
    ids = [3, 49, 0, 17]
    SurfaceIO.writeEmbeddingBatchFP16(s, 0, spatial, table, vocab, dim, ids)
    got = SurfaceIO.readFP16(s, 0, dim, spatial)
    for lane, t in enumerate(ids):
        assert np.array_equal(got[:, lane], table[t].astype(np.float16).astype(np.float32))
    assert np.all(got[:, len(ids):] == 0)
    with pytest.raises(io.SurfaceIOError):
        SurfaceIO.writeEmbeddingBatchFP16(s, 0, spatial, table, vocab, dim, [50])
    idx, val = SurfaceIO.argmaxBatchFP16Spatial(s, 0, spatial, dim, 4)
    assert idx == [int(np.argmax(got[:, l])) for l in range(4)]
    assert val == [float(got[:, l].max()) for l in range(4)]


def test_lock_unlock_and_unlocked_io():           # SurfaceIO.swift:720-781
    L = io._L()
    s = Surface.create(64)
    x = np.arange(32, dtype=np.float32)
    out = np.empty(32, np.float32)
    assert not L.esp_interop_io_write_fp16_unlocked(s.ref, x.ctypes.data_as(C.c_void_p), 32, 1)     # needs the lock
    assert not L.esp_interop_io_unlock_write(s.ref)
    assert L.esp_interop_io_lock_write(s.ref)
    assert L.esp_interop_io_write_fp16_unlocked(s.ref, x.ctypes.data_as(C.c_void_p), 32, 1)
    assert L.esp_interop_io_unlock_write(s.ref)
    assert L.esp_interop_io_lock_read(s.ref)
    assert L.esp_interop_io_read_fp16_unlocked(s.ref, 0, out.ctypes.data_as(C.c_void_p), 32, 1)
    assert L.esp_interop_io_unlock_read(s.ref) and not L.esp_interop_io_unlock_read(s.ref)
    assert np.array_equal(out, x)


def test_retain_release_counts():
    L = io._L()
    ref = L.esp_interop_create_surface(32)
    assert L.esp_surface_retain(ref) == ref
    L.esp_surface_release(ref)
    assert L.esp_surface_bytes(ref) == 32        # still alive after one of two releases
    L.esp_surface_release(ref)
