"""esp_gemv_device_noalloc: the GEMV entry point that allocates nothing, against esp_gemv.

The caller owns the device buffers; here they come straight from the HIP runtime the library is linked with.
Two calls in a row share the library's fixed scratch array, the second with a smaller input."""
import ctypes as C

import numpy as np
import pytest

from oracle import oracle as orc

pytestmark = pytest.mark.gpu


class DeviceBuffer:
    """hipMalloc'ed memory owned by the test (the entry point under test must not allocate)."""

    def __init__(self, hip, nbytes):
        self.hip, self.nbytes, self.ptr = hip, nbytes, C.c_void_p()
        assert hip.hipMalloc(C.byref(self.ptr), C.c_size_t(nbytes)) == 0

    def upload(self, a):
        a = np.ascontiguousarray(a)
        assert a.nbytes <= self.nbytes
        assert self.hip.hipMemcpy(self.ptr, a.ctypes.data_as(C.c_void_p), C.c_size_t(a.nbytes), 1) == 0   # host to device

    def download(self, shape, dtype):
        out = np.empty(shape, dtype)
        assert out.nbytes <= self.nbytes
        assert self.hip.hipMemcpy(out.ctypes.data_as(C.c_void_p), self.ptr, C.c_size_t(out.nbytes), 2) == 0  # device to host
        return out

    def free(self):
        self.hip.hipFree(self.ptr)


@pytest.fixture(scope="module")
def env():
    import espresso_amd._lib as lib
    import espresso_amd.ops as ops
    ops.init()
    hip = C.CDLL("libamdhip64.so")      # the runtime libespresso_hip.so already loaded
    hip.hipMalloc.argtypes = [C.POINTER(C.c_void_p), C.c_size_t]
    hip.hipMemcpy.argtypes = [C.c_void_p, C.c_void_p, C.c_size_t, C.c_int]
    hip.hipFree.argtypes = [C.c_void_p]
    L = lib.load_library()
    L.esp_gemv_device_noalloc.restype = C.c_int
    L.esp_gemv_device_noalloc.argtypes = [C.c_void_p, C.c_void_p, C.c_int, C.c_void_p, C.c_void_p]
    return lib, ops, hip, L


def run_noalloc(env, mat, x, residual=None):
    lib, ops, hip, L = env
    batch = x.shape[0]
    dx, dy = DeviceBuffer(hip, x.nbytes), DeviceBuffer(hip, batch * mat.rows * 4)
    dr = DeviceBuffer(hip, batch * mat.rows * 4) if residual is not None else None
    dx.upload(x)
    dy.upload(np.full((batch, mat.rows), np.nan, np.float32))
    if dr:
        dr.upload(residual)
    lib.check(L.esp_gemv_device_noalloc(mat._h, dx.ptr, batch, dy.ptr, dr.ptr if dr else None))
    y = dy.download((batch, mat.rows), np.float32)
    for b in (dx, dy, dr):
        if b:
            b.free()
    return y


def make_matrix(ops, fmt, rows, cols, seed):
    w = np.random.default_rng(seed).normal(0, 0.05, (rows, cols)).astype(np.float32)
    return ops.Matrix(fmt, orc.quantize(fmt, w), rows, cols)


def test_two_calls_in_a_row_share_the_scratch_and_match_esp_gemv(env):
    lib, ops, hip, L = env
    rng = np.random.default_rng(1)
    # first call: Q8_0 768 x 2048 at batch 16 (register-B MFMA kernel, K split four ways: partial sums in the scratch)
    big = make_matrix(ops, orc.FMT_Q8_0, 768, 2048, 2)
    x1 = rng.normal(0, 1, (16, 2048)).astype(np.float16)
    r1 = rng.normal(0, 1, (16, 768)).astype(np.float32)
    y1 = run_noalloc(env, big, x1, r1)
    # second call, smaller, over whatever the first left in the scratch
    small = make_matrix(ops, orc.FMT_Q8_0, 256, 1024, 3)
    x2 = rng.normal(0, 1, (5, 1024)).astype(np.float16)
    y2 = run_noalloc(env, small, x2)
    # the same kernels, the same split counts, the same order of additions: bit for bit what esp_gemv returns
    assert np.array_equal(y1.view(np.uint32), big.gemv(x1, r1).view(np.uint32))
    assert np.array_equal(y2.view(np.uint32), small.gemv(x2).view(np.uint32))
    # and the first call again after the second
    assert np.array_equal(run_noalloc(env, big, x1, r1).view(np.uint32), y1.view(np.uint32))
    # against the oracle's matvec on the dequantised weights (MFMA path: weights rounded to fp16 once)
    deq = big.dequantize()
    want = np.stack([orc.matvec(deq, x1[b].astype(np.float32)) for b in range(16)]) + r1
    assert np.abs(y1 - want).max() <= 1e-3 * np.abs(deq).max() * np.sqrt(2048) * 4
    big.close(); small.close()


@pytest.mark.parametrize("fmt,rows,cols,batch", [
    (orc.FMT_Q4_K, 512, 1024, 1), (orc.FMT_Q4_K, 512, 1024, 2), (orc.FMT_Q4_K, 512, 1024, 8), (orc.FMT_Q4_0, 256, 16384, 6),
    (orc.FMT_F16, 384, 512, 40), (orc.FMT_Q8_0, 32000, 768, 64),
])
def test_formats_and_batches_match_esp_gemv(env, fmt, rows, cols, batch):
    lib, ops, hip, L = env
    mat = make_matrix(ops, fmt, rows, cols, rows + cols)
    x = np.random.default_rng(batch).normal(0, 1, (batch, cols)).astype(np.float16)
    assert np.array_equal(run_noalloc(env, mat, x).view(np.uint32), mat.gemv(x).view(np.uint32))
    mat.close()


def test_sizes_beyond_the_fixed_scratch_are_refused(env):
    lib, ops, hip, L = env
    mat = make_matrix(ops, orc.FMT_Q8_0, 64, 256, 9)
    d = DeviceBuffer(hip, 1 << 20)
    with pytest.raises(lib.EspressoError, match="batch 65 outside 1..64"):
        lib.check(L.esp_gemv_device_noalloc(mat._h, d.ptr, 65, d.ptr, None))
    with pytest.raises(lib.EspressoError, match="null pointer"):
        lib.check(L.esp_gemv_device_noalloc(mat._h, None, 1, d.ptr, None))
    mat.close()
    # 40000 rows x batch 64 would need 5.1 M floats for two splits
    tall = ops.Matrix(orc.FMT_F16, np.zeros(40000 * 64 * 2, np.uint8), 40000, 64)
    with pytest.raises(lib.EspressoError, match="fixed scratch holds"):
        lib.check(L.esp_gemv_device_noalloc(tall._h, d.ptr, 64, d.ptr, None))
    tall.close()
    d.free()
