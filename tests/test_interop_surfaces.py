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


def test_two_slice_copy_checks_both_pairs_before_touching_either():   # SurfaceIO.swift:285-339
    channels = 6
    k_src, v_src = Surface.create(channels * 4 * 2), Surface.create(channels * 4 * 2)
    k_dst, v_dst = Surface.create(channels * 16 * 2), Surface.create(channels * 16 * 2)
    rng = np.random.default_rng(21)
    k, v = rng.normal(0, 1, (channels, 4)).astype(np.float32), rng.normal(0, 1, (channels, 4)).astype(np.float32)
    SurfaceIO.writeFP16(k_src, k, channels, 4)
    SurfaceIO.writeFP16(v_src, v, channels, 4)
    SurfaceIO.copyTwoFP16SpatialSlices(k_dst, 0, 9, 16, k_src, 0, 2, 4, v_dst, 0, 9, 16, v_src, 0, 1, 4, channels)
    assert np.array_equal(SurfaceIO.readFP16SpatialSlice(k_dst, 0, 9, 16, channels), k[:, 2].astype(np.float16).astype(np.float32))
    assert np.array_equal(SurfaceIO.readFP16SpatialSlice(v_dst, 0, 9, 16, channels), v[:, 1].astype(np.float16).astype(np.float32))
    with pytest.raises(io.SurfaceIOError):          # the second pair is out of range: the first must stay untouched
        SurfaceIO.copyTwoFP16SpatialSlices(k_dst, 0, 3, 16, k_src, 0, 0, 4, v_dst, 0, 16, 16, v_src, 0, 0, 4, channels)
    assert np.all(SurfaceIO.readFP16SpatialSlice(k_dst, 0, 3, 16, channels) == 0)


def test_batched_writes_and_copies_are_all_or_nothing():   # SurfaceIO.swift:190-229, :672-716, :783-828
    channels, spatial = 12, 4
    s, t, u = (Surface.create(channels * spatial * 2) for _ in range(3))
    a, b = np.arange(2 * spatial, dtype=np.float32) + 1, -(np.arange(3 * spatial, dtype=np.float32) + 1)
    SurfaceIO.writeFP16AtBatched(s, spatial, [(1, a, 2), (7, b, 3)])
    got = SurfaceIO.readFP16(s, 0, channels, spatial)
    assert np.array_equal(got[1:3].ravel(), a) and np.array_equal(got[7:10].ravel(), b)
    assert np.all(got[0] == 0) and np.all(got[3:7] == 0) and np.all(got[10:] == 0)
    with pytest.raises(io.SurfaceIOError):          # second region runs past the surface: nothing is written
        SurfaceIO.writeFP16AtBatched(t, spatial, [(0, a, 2), (10, b, 3)])
    assert np.all(SurfaceIO.readFP16(t, 0, channels, spatial) == 0)
    SurfaceIO.copyFP16Batched(t, s, spatial, [(0, 7, 3), (5, 1, 2)])
    got_t = SurfaceIO.readFP16(t, 0, channels, spatial)
    assert np.array_equal(got_t[0:3], got[7:10]) and np.array_equal(got_t[5:7], got[1:3]) and np.all(got_t[3:5] == 0) and np.all(got_t[7:] == 0)
    with pytest.raises(io.SurfaceIOError):
        SurfaceIO.copyFP16Batched(u, s, spatial, [(0, 7, 3), (11, 1, 2)])
    assert np.all(SurfaceIO.readFP16(u, 0, channels, spatial) == 0)
    SurfaceIO.copyFP16FromMultipleSources(u, spatial, [(s, 0, 1, 2), (t, 4, 0, 3), (s, 9, 7, 3)])
    got_u = SurfaceIO.readFP16(u, 0, channels, spatial)
    assert np.array_equal(got_u[0:2], got[1:3]) and np.array_equal(got_u[4:7], got_t[0:3]) and np.array_equal(got_u[9:12], got[7:10])
    with pytest.raises(io.SurfaceIOError):
        SurfaceIO.copyFP16FromMultipleSources(u, spatial, [(s, 0, 1, 2), (t, 4, 11, 3)])
    SurfaceIO.copyFP16Batched(u, s, spatial, [])    # empty region lists are no-ops (SurfaceIO.swift:676, :787)
    SurfaceIO.copyFP16FromMultipleSources(u, spatial, [])


def test_block_partitioned_argmax_is_the_serial_first_maximum():   # surface_io.c:689-700; SurfaceIO.swift:542-615
    channels, spatial, streams = 1003, 8, 5
    rng = np.random.default_rng(33)
    x = rng.normal(0, 1, (channels, spatial)).astype(np.float32)
    x[[250, 251, 600], 0] = 9.0                     # ties across every block boundary of the partitions below
    x[[1002, 17], 1] = 7.5                          # the first and the last block
    x[:, 2] = -3.0                                  # all equal: channel 0
    x[:, 3] = -65504.0                              # the lowest finite value everywhere
    s = Surface.create((channels + 4) * spatial * 2)
    SurfaceIO.writeFP16At(s, 4, x, channels, spatial)
    serial = SurfaceIO.argmaxBatchFP16Spatial(s, 4, spatial, channels, streams)
    assert serial[0][:4] == [250, 17, 0, 0] and serial[1][:4] == [9.0, 7.5, -3.0, -65504.0]
    for blocks in (1, 2, 3, 4, 7, 8, 16, 1003, 5000):
        assert SurfaceIO.argmaxBatchFP16SpatialParallel(s, 4, spatial, channels, streams, blocks) == serial
        assert SurfaceIO.argmaxBatchFP16SpatialNolock(s, 4, spatial, channels, streams, blocks) == serial
    with pytest.raises(io.SurfaceIOError):
        SurfaceIO.argmaxBatchFP16SpatialParallel(s, 4, spatial, channels + 1, streams, 4)
    with pytest.raises(io.SurfaceIOError):
        SurfaceIO.argmaxBatchFP16SpatialParallel(s, 4, spatial, channels, spatial + 1, 4)


def test_argmax_with_hint_is_the_first_maximum_and_survives_a_wrong_hint():   # SurfaceIO.swift:433-474
    channels, spatial = 300, 4
    rng = np.random.default_rng(34)
    x = rng.normal(0, 1, (channels, spatial)).astype(np.float32)
    x[[40, 200], 1] = 6.0
    s, hint = Surface.create(channels * spatial * 2), Surface.create(spatial * 2)
    SurfaceIO.writeFP16(s, x, channels, spatial)
    SurfaceIO.writeFP16(hint, x.astype(np.float16).astype(np.float32).max(axis=0), 1, spatial)
    for lane in range(spatial):
        assert SurfaceIO.argmaxFP16SpatialSliceWithHint(s, 0, lane, spatial, channels, hint, lane, spatial) == SurfaceIO.argmaxFP16SpatialSlice(s, 0, lane, spatial, channels)
    assert SurfaceIO.argmaxFP16SpatialSliceWithHint(s, 0, 1, spatial, channels, hint, 1, spatial) == (40, 6.0)
    # a hint that matches no channel (lane 1's maximum used for lane 0) still gives the scan's answer
    assert SurfaceIO.argmaxFP16SpatialSliceWithHint(s, 0, 0, spatial, channels, hint, 1, spatial) == SurfaceIO.argmaxFP16SpatialSlice(s, 0, 0, spatial, channels)
    with pytest.raises(io.SurfaceIOError):
        SurfaceIO.argmaxFP16SpatialSliceWithHint(s, 0, 0, spatial, channels, hint, spatial, spatial)


def test_strided_gather_and_scatter_convert_like_the_contiguous_routines():   # ane_interop.h:160, :165
    rng = np.random.default_rng(35)
    x = rng.normal(0, 2, 96).astype(np.float32)
    bits = io.cvt_f32_to_f16(x)
    assert np.array_equal(io.gather_f16_to_f32(bits, 12, 8), io.cvt_f16_to_f32(bits[::8]))
    dst = np.full(96, 0x7BFF, np.uint16)
    io.scatter_f32_to_f16(dst, x[:12], 8)
    assert np.array_equal(dst[::8], io.cvt_f32_to_f16(x[:12]))
    untouched = np.ones(96, bool); untouched[::8] = False
    assert np.all(dst[untouched] == 0x7BFF)


def test_fused_expansion_argmax_follows_fp16_fused_multiply_adds():   # surface_io.c:1438-1700
    """Parity unpinned against the reference (it holds no vector for this routine); pinned here against exact
    fp16 arithmetic done in numpy: every term is one fused multiply-add rounded to fp16, terms in channel order."""
    bottleneck, groups, vocab, spatial, streams = 32, 4, 96, 8, 3
    cpg, per = bottleneck // groups, vocab // groups
    rng = np.random.default_rng(36)
    proj = rng.normal(0, 1, (bottleneck, spatial)).astype(np.float16)
    w = rng.normal(0, 1, (vocab, cpg)).astype(np.float16)
    w[50] = w[49]                                   # rows 49 and 50 (same group) tie exactly: 49 wins whenever they lead
    s = Surface.create((bottleneck + 2) * spatial * 2)
    SurfaceIO.writeFP16At(s, 2, proj.astype(np.float32), bottleneck, spatial)
    want_i, want_v = [], []
    for lane in range(streams):
        logits = np.empty(vocab, np.float16)
        for c in range(vocab):
            g, acc = c // per, np.float16(0)
            for k in range(cpg):
                acc = np.float16(np.float64(w[c, k]) * np.float64(proj[g * cpg + k, lane]) + np.float64(acc))
            logits[c] = acc
        want_i.append(int(np.argmax(logits))); want_v.append(float(logits.max()))
    got_i, got_v = SurfaceIO.fusedExpansionArgmax(s, 2, spatial, bottleneck, groups, w.view(np.uint16), vocab, streams)
    assert got_i == want_i and got_v == want_v
    # a one-hot projection selects one weight column: the winner is that column's largest entry within the group
    onehot = np.zeros((bottleneck, spatial), np.float32); onehot[cpg * 2 + 3, 0] = 1.0
    SurfaceIO.writeFP16At(s, 2, onehot, bottleneck, spatial)
    col = w[2 * per:3 * per, 3].astype(np.float32)
    i, v = SurfaceIO.fusedExpansionArgmax(s, 2, spatial, bottleneck, groups, w.view(np.uint16), vocab, 1)
    if col.max() > 0:
        assert i == [2 * per + int(np.argmax(col))] and v == [float(col.max())]
    else:
        assert v == [0.0]                             # every other group scores exactly 0
    # the reference's argument checks
    for bad in (dict(spatial=12), dict(vocab=65536 + 32), dict(groups=5), dict(streams=spatial + 1)):
        sp, vc, gr, st = bad.get("spatial", spatial), bad.get("vocab", vocab), bad.get("groups", groups), bad.get("streams", streams)
        idx, val = (C.c_int * 16)(), (C.c_float * 16)()
        assert not io._L().esp_interop_fused_expansion_argmax_fp16(s.ref, 2, sp, bottleneck, gr, w.ctypes.data_as(C.c_void_p), vc, st, idx, val, 4)
