"""GPU parity: GGUF block dequantisation (bit-exact) and the dequant-fused GEMV (tolerance) against
the CPU oracle, through the C ABI."""
import numpy as np
import pytest

from oracle import oracle as orc

pytestmark = pytest.mark.gpu

FORMATS = {"q8_0": (orc.FMT_Q8_0, 34, 32), "q4_0": (orc.FMT_Q4_0, 18, 32), "q4_k": (orc.FMT_Q4_K, 144, 256),
           "f16": (orc.FMT_F16, 2, 1), "f32": (orc.FMT_F32, 4, 1)}


def _bits(a):
    return np.ascontiguousarray(a, dtype=np.float32).view(np.uint32)


@pytest.fixture(scope="module")
def ops():
    import espresso_amd.ops as o
    o.init()
    return o


@pytest.mark.parametrize("name", ["q8_0", "q4_0", "q4_k", "f16"])
def test_dequantize_random_bytes_bit_exact(ops, name):
    fmt, blk_bytes, blk_len = FORMATS[name]
    rng = np.random.default_rng(fmt + 100)
    nb = 8192 if blk_len > 1 else 65536
    blocks = rng.integers(0, 256, nb * blk_bytes, dtype=np.uint8)
    if blk_len > 1:   # edge scales: 0, -0, smallest subnormal, largest finite, inf, largest subnormal, smallest normal
        for i, e in enumerate([0x0000, 0x8000, 0x0001, 0x7BFF, 0x7C00, 0x03FF, 0x0400, 0xFBFF]):
            blocks[i * blk_bytes:i * blk_bytes + 2] = np.array([e], np.uint16).view(np.uint8)
    want = orc.dequantize(fmt, blocks, nb * blk_len)
    got = ops.dequantize(fmt, blocks, nb * blk_len)
    nan = np.isnan(want)
    assert np.array_equal(np.isnan(got), nan)
    assert np.array_equal(_bits(got)[~nan], _bits(want)[~nan])


def test_dequantize_q4_k_exhaustive_scale_min_nibble(ops):
    blocks = []
    for d, dmin in [(0.0123, 0.0456), (6.1e-5, 5.96e-8), (-0.37, 3.3e-4)]:
        for sc in range(64):
            for m0 in range(0, 64, 8):
                blk = np.zeros(144, np.uint8)
                blk[0:2] = np.array([d], np.float16).view(np.uint8)
                blk[2:4] = np.array([dmin], np.float16).view(np.uint8)
                scs = np.full(8, sc); ms = m0 + np.arange(8)
                for j in range(4):
                    blk[4 + j] = scs[j] | ((scs[j + 4] >> 4) << 6)
                    blk[8 + j] = ms[j] | ((ms[j + 4] >> 4) << 6)
                    blk[12 + j] = (scs[j + 4] & 0xF) | ((ms[j + 4] & 0xF) << 4)
                nib = (np.arange(256) % 16).astype(np.uint8)
                for c in range(4):
                    blk[16 + 32 * c:16 + 32 * c + 32] = nib[64 * c:64 * c + 32] | (nib[64 * c + 32:64 * c + 64] << 4)
                blocks.append(blk)
    blocks = np.concatenate(blocks)
    n = blocks.size // 144 * 256
    assert np.array_equal(_bits(ops.dequantize(orc.FMT_Q4_K, blocks, n)), _bits(orc.dequantize(orc.FMT_Q4_K, blocks, n)))


def test_dequantize_edge_arguments(ops):
    import espresso_amd._lib as lib
    assert ops.dequantize(orc.FMT_Q8_0, np.zeros(0, np.uint8), 0).size == 0       # empty tensor
    with pytest.raises(lib.EspressoError):
        ops.dequantize(orc.FMT_Q4_K, np.zeros(144, np.uint8), 100)                # ragged element count
    with pytest.raises(lib.EspressoError):
        ops.dequantize(7, np.zeros(144, np.uint8), 256)                           # unknown format


def _quantized(fmt, rows, cols, seed):
    rng = np.random.default_rng(seed)
    w = rng.normal(0, 0.02, (rows, cols)).astype(np.float32)
    blocks = orc.quantize(fmt, w)
    return blocks, orc.dequantize(fmt, blocks, rows * cols).reshape(rows, cols)


@pytest.mark.parametrize("name,rows,cols", [
    ("q8_0", 768, 768), ("q8_0", 2048, 768), ("q8_0", 768, 2048), ("q8_0", 1003, 96),
    ("q4_0", 1024, 4096), ("q4_0", 515, 256), ("q4_k", 1024, 4096), ("q4_k", 257, 1024), ("q4_k", 64, 14336),
    ("q4_k", 515, 2048), ("q4_k", 300, 8192), ("q4_k", 131, 11008), ("q4_k", 6000, 4096),
    ("f16", 768, 768), ("f16", 333, 2048), ("f32", 301, 512),
])
@pytest.mark.parametrize("batch", [1, 2])
def test_gemv_matches_oracle(ops, name, rows, cols, batch):
    fmt = FORMATS[name][0]
    blocks, deq = _quantized(fmt, rows, cols, seed=rows * 7 + cols + batch)
    rng = np.random.default_rng(rows + cols)
    x = rng.normal(0, 1, (batch, cols)).astype(np.float16)
    mat = ops.Matrix(fmt, blocks, rows, cols)
    # the resident layout decodes to the same bits as the GGUF blocks
    assert np.array_equal(_bits(mat.dequantize()), _bits(deq))
    y = mat.gemv(x)
    want = np.stack([orc.matvec(deq, x[b].astype(np.float32)) for b in range(batch)])
    # fp32 accumulation on both sides; only the summation order differs.
    scale = np.abs(deq).max() * np.sqrt(cols)
    assert np.abs(y - want).max() <= 2e-5 * scale + 1e-6, np.abs(y - want).max()
    # fused residual epilogue
    res = rng.normal(0, 1, (batch, rows)).astype(np.float32)
    y2 = mat.gemv(x, residual=res)
    assert np.abs(y2 - (res + want)).max() <= 2e-5 * scale + 1e-6
    mat.close()


def test_gemv_special_inputs(ops):
    fmt = orc.FMT_Q4_K
    blocks, deq = _quantized(fmt, 64, 512, seed=5)
    mat = ops.Matrix(fmt, blocks, 64, 512)
    # zero activations give exactly zero; a one-hot picks a column of the dequantised matrix
    assert np.array_equal(mat.gemv(np.zeros((1, 512), np.float16)), np.zeros((1, 64), np.float32))
    for col in (0, 17, 255, 256, 300, 511):
        e = np.zeros((1, 512), np.float16); e[0, col] = 1
        assert np.allclose(mat.gemv(e)[0], deq[:, col], rtol=0, atol=1e-7)
    # linearity in x (property that holds at any size)
    rng = np.random.default_rng(9)
    a, b = rng.normal(0, 1, (1, 512)).astype(np.float16), rng.normal(0, 1, (1, 512)).astype(np.float16)
    s = (a.astype(np.float32) + b.astype(np.float32)).astype(np.float16)
    exact = (s.astype(np.float32) == a.astype(np.float32) + b.astype(np.float32)).all()
    if exact:
        assert np.allclose(mat.gemv(s), mat.gemv(a) + mat.gemv(b), atol=1e-5)
    mat.close()


def test_gemv_argument_errors(ops):
    import espresso_amd._lib as lib
    with pytest.raises(ValueError):
        ops.Matrix(orc.FMT_Q4_K, np.zeros(100, np.uint8), 4, 256)                 # wrong byte count
    with pytest.raises(ValueError):
        ops.Matrix(orc.FMT_Q4_K, np.zeros(144, np.uint8), 1, 100)                 # ragged cols
    with pytest.raises(ValueError):
        ops.Matrix(7, np.zeros(4 * 64, np.uint8), 1, 64)                          # unknown format


@pytest.mark.parametrize("name,rows,cols", [
    ("q4_k", 1024, 4096), ("q4_k", 200, 1024), ("q4_k", 256, 14336), ("q8_0", 768, 768), ("q8_0", 1003, 2048),
    ("q4_0", 515, 256), ("q4_0", 1024, 4096), ("f16", 333, 2048),
])
@pytest.mark.parametrize("batch", [3, 8, 32, 33, 64, 100, 130])
def test_mfma_gemm_matches_oracle(ops, name, rows, cols, batch):
    """More than two activation rows run the dequant-fused MFMA kernel: fp16 weights (one rounding of the
    dequantised value), fp32 accumulation; compared per row with the oracle's fp32 matvec."""
    fmt = FORMATS[name][0]
    blocks, deq = _quantized(fmt, rows, cols, seed=rows + 3 * cols)
    rng = np.random.default_rng(batch * 1000 + rows)
    x = rng.normal(0, 1, (batch, cols)).astype(np.float16)
    mat = ops.Matrix(fmt, blocks, rows, cols)
    y = mat.gemv(x)
    check = [0, 1, batch // 2, batch - 2, batch - 1]
    want = np.stack([orc.matvec(deq, x[b].astype(np.float32)) for b in check])
    # each weight carries one fp16 rounding (2^-11 relative): random-sign errors over cols terms
    tol = 2.0 ** -11 * np.abs(deq).max() * 4.0 * np.sqrt(cols) + 1e-5
    assert np.abs(y[check] - want).max() <= tol, (np.abs(y[check] - want).max(), tol)
    # every format feeds the matrix cores fp16(dequantised weight), rounded once: against those weights in
    # float64 only fp32 summation noise remains (pins the tile indexing and the single rounding)
    # (up to eight rows against Q4_K and Q4_0 run on the nibbles themselves with exact products: no weight rounding at all)
    exact = batch <= 8 and cols % 256 == 0 and (name == "q4_k" or (name == "q4_0" and cols <= 8192))
    ref = x.astype(np.float64) @ (deq if exact else deq.astype(np.float16)).astype(np.float64).T
    assert np.abs(y - ref).max() <= 2e-5 * np.abs(deq).max() * np.sqrt(cols) * 4 + 1e-6, np.abs(y - ref).max()
    res = rng.normal(0, 1, (batch, rows)).astype(np.float32)
    y2 = mat.gemv(x, residual=res)
    assert np.abs(y2 - (res + y)).max() <= 1e-5 * (1 + np.abs(y).max())
    mat.close()
