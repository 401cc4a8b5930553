"""GPU parity for the kernel-handle API: each kernel kind is compiled from program text, fed through its
input surface and compared with the CPU oracle's restatement of the reference generator it stands for."""
import numpy as np
import pytest

from oracle import oracle as orc

pytestmark = pytest.mark.gpu

FMT = {"q8_0": orc.FMT_Q8_0, "q4_0": orc.FMT_Q4_0, "q4_k": orc.FMT_Q4_K, "f16": orc.FMT_F16}


@pytest.fixture(scope="module")
def io():
    import espresso_amd.interop as m
    import espresso_amd.ops as o
    o.init()
    return m


def _f16(a):
    return np.asarray(a, dtype=np.float32).astype(np.float16).astype(np.float32)


def _matrix(name, rows, cols, rng):
    w = rng.normal(0, 0.02, (rows, cols)).astype(np.float32)
    if name == "f16":
        return orc.blob_build(w), _f16(w)
    blocks = orc.quantize(FMT[name], w)
    return blocks.tobytes(), orc.dequantize(FMT[name], blocks, rows * cols).reshape(rows, cols)


def _fp16_close(got, want, extra=0.0):
    # one fp16 rounding of the result plus fp32 summation-order noise
    tol = np.abs(want) * 2.0 ** -10 + 1e-4 + extra
    assert np.all(np.abs(got - want) <= tol), float(np.abs(got - want).max())


@pytest.mark.parametrize("name,rows,cols,spatial,lanes", [("q8_0", 768, 768, 32, 1), ("q4_k", 512, 1024, 8, 4), ("q4_0", 96, 256, 1, 1), ("f16", 200, 320, 16, 16)])
def test_gemv_kernel_matches_oracle(io, name, rows, cols, spatial, lanes):
    rng = np.random.default_rng(rows + cols)
    blob, deq = _matrix(name, rows, cols, rng)
    before = io._L().esp_interop_compile_count()
    k = io.ANEKernel(io.program_text("gemv", name, spatial, lanes, rows=rows, cols=cols), [("@model_path/weights/w.bin", blob)],
                     [cols * spatial * 2], [rows * spatial * 2])
    assert io._L().esp_interop_compile_count() == before + 1 and io._L().esp_interop_live_handle_count() == 1
    x = rng.normal(0, 1, (cols, spatial)).astype(np.float32)
    xin, out = k.inputSurface(0), k.outputSurface(0)
    io.SurfaceIO.writeFP16(xin, x, cols, spatial)
    k.eval()
    got = io.SurfaceIO.readFP16(out, 0, rows, spatial)
    for lane in range(lanes):
        _fp16_close(got[:, lane], orc.matvec(deq, _f16(x[:, lane])))
    assert np.all(got[:, lanes:] == 0)                       # columns past `lanes` are never written
    assert k.lastHWExecutionTimeNS() > 0
    # a second eval after rewriting one column only changes that column
    col = rng.normal(0, 1, cols).astype(np.float32)
    io.SurfaceIO.writeFP16SpatialSlice(xin, 0, 0, spatial, col, cols)
    k.eval()
    got2 = io.SurfaceIO.readFP16(out, 0, rows, spatial)
    _fp16_close(got2[:, 0], orc.matvec(deq, _f16(col)))
    assert np.array_equal(got2[:, 1:], got[:, 1:])
    k.free()
    assert io._L().esp_interop_live_handle_count() == 0


def test_rmsnorm_classifier_kernel_matches_oracle(io):
    dim, vocab, spatial, lanes = 256, 4000, 8, 3
    rng = np.random.default_rng(1)
    blob, deq = _matrix("q8_0", vocab, dim, rng)
    gamma = (1.0 + rng.normal(0, 0.1, dim)).astype(np.float32)
    k = io.ANEKernel(io.program_text("rmsnorm_classifier", "q8_0", spatial, lanes, dim=dim, vocab=vocab),
                     [("@model_path/weights/rms_final.bin", orc.blob_build(gamma)), ("@model_path/weights/classifier.bin", blob)],
                     [dim * spatial * 2], [vocab * spatial * 2, spatial * 2])
    x = rng.normal(0, 1, (dim, spatial)).astype(np.float32)
    io.SurfaceIO.writeFP16(k.inputSurface(0), x, dim, spatial)
    k.eval()
    logits = io.SurfaceIO.readFP16(k.outputSurface(0), 0, vocab, spatial)
    mx = io.SurfaceIO.readFP16(k.outputSurface(1), 0, 1, spatial)
    for lane in range(lanes):
        n = _f16(orc.rmsnorm(_f16(x[:, lane]), _f16(gamma), 1e-5))
        want = orc.matvec(deq, n)
        _fp16_close(logits[:, lane], want, extra=2e-3)
        assert abs(mx[0, lane] - want.max()) <= abs(want.max()) * 2.0 ** -10 + 2e-3
        # the surface argmax agrees with the oracle's whenever the top-2 margin exceeds the fp16 step
        top = np.sort(want)[-2:]
        if top[1] - top[0] > 4e-3:
            assert io.SurfaceIO.argmaxFP16SpatialSlice(k.outputSurface(0), 0, lane, spatial, vocab)[0] == int(np.argmax(want))
    k.free()


@pytest.mark.parametrize("name,dim,hidden", [("q8_0", 768, 2048), ("q4_k", 512, 1024), ("q4_k", 2048, 8192), ("q4_k", 4096, 11008)])
def test_decode_ffn_kernel_matches_oracle(io, name, dim, hidden):
    spatial, lanes = 32, 2
    rng = np.random.default_rng(dim)
    b1, w1 = _matrix(name, hidden, dim, rng)
    b3, w3 = _matrix(name, hidden, dim, rng)
    b2, w2 = _matrix(name, dim, hidden, rng)
    gamma = (1.0 + rng.normal(0, 0.1, dim)).astype(np.float32)
    k = io.ANEKernel(io.program_text("decode_ffn", name, spatial, lanes, dim=dim, hidden=hidden),
                     [("@model_path/weights/rms_ffn.bin", orc.blob_build(gamma)), ("@model_path/weights/w1.bin", b1),
                      ("@model_path/weights/w3.bin", b3), ("@model_path/weights/w2.bin", b2)], [dim * spatial * 2], [dim * spatial * 2])
    x = rng.normal(0, 1, (dim, spatial)).astype(np.float32)
    io.SurfaceIO.writeFP16(k.inputSurface(0), x, dim, spatial)
    k.eval()
    got = io.SurfaceIO.readFP16(k.outputSurface(0), 0, dim, spatial)
    for lane in range(lanes):
        xl = _f16(x[:, lane])
        n = _f16(orc.rmsnorm(xl, _f16(gamma), 1e-5))
        g, u = orc.matvec(w1, n), orc.matvec(w3, n)
        act = _f16(np.array([orc.silu_tanh(float(v)) for v in g], dtype=np.float32) * u)
        want = xl + orc.matvec(w2, act)
        # the fp16 rounding of the hidden activations adds noise that grows with the number of terms of the down projection
        _fp16_close(got[:, lane], want, extra=1e-3 * max(1.0, hidden / 2048))
    k.free()


def test_compile_errors_eval_failure_hook_and_rebind(io):
    L = io._L()
    rng = np.random.default_rng(3)
    blob, deq = _matrix("q8_0", 64, 64, rng)
    before = L.esp_interop_compile_count()
    with pytest.raises(io.ANEError, match="compilationFailed"):      # not a program this library knows
        io.ANEKernel("this is not a program", [], [64], [64])
    with pytest.raises(io.ANEError, match="compilationFailed"):      # weight missing
        io.ANEKernel(io.program_text("gemv", "q8_0", rows=64, cols=64), [], [128], [128])
    with pytest.raises(io.ANEError, match="compilationFailed"):      # weight bytes do not match rows x cols
        io.ANEKernel(io.program_text("gemv", "q8_0", rows=64, cols=128), [("w.bin", blob)], [256], [128])
    with pytest.raises(io.ANEError, match="invalidArguments"):       # surface size does not match the program
        io.ANEKernel(io.program_text("gemv", "q8_0", rows=64, cols=64), [("w.bin", blob)], [64], [128])
    assert L.esp_interop_compile_count() == before and L.esp_interop_live_handle_count() == 0
    k = io.ANEKernel(io.program_text("gemv", "q8_0", rows=64, cols=64), [("w.bin", blob)], [128], [128])
    L.esp_interop_set_force_eval_failure(True)
    try:
        with pytest.raises(io.ANEError, match="evaluationFailed"):
            k.eval()
    finally:
        L.esp_interop_set_force_eval_failure(False)
    # rebinding the input to a caller-made surface
    mine = io.Surface.create(128)
    x = rng.normal(0, 1, 64).astype(np.float32)
    io.SurfaceIO.writeFP16(mine, x, 64, 1)
    k.rebindInput(0, mine)
    k.eval()
    _fp16_close(io.SurfaceIO.readFP16(k.outputSurface(0), 0, 64, 1)[:, 0], orc.matvec(deq, _f16(x)))
    with pytest.raises(io.ANEError):
        k.rebindInput(0, io.Surface.create(64))                      # wrong size
    k.free()
