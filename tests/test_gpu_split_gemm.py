"""The Q4_K block GEMM that rounds no operand (esp_matmul_f32: fp32 activations as hi / lo fp16 pairs, weights as the exact
integers sc * q with d, dmin and the minimums applied in fp32) against float64 products of the oracle's dequantised weights."""
import numpy as np
import pytest

from oracle import oracle as orc

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ops():
    import espresso_amd.ops as o
    o.init()
    return o


def q4k(ops, rows, cols, seed):
    w = np.random.default_rng(seed).normal(0, 0.02, (rows, cols)).astype(np.float32)
    blocks = orc.quantize(orc.FMT_Q4_K, w)
    deq = orc.dequantize(orc.FMT_Q4_K, blocks, rows * cols).reshape(rows, cols)
    return ops.Matrix(orc.FMT_Q4_K, blocks, rows, cols), deq


# (weight rows, columns, activation rows): one tile, ragged in both directions, K split over the grid (few workgroups), the 8B
# projections at a full 512-row block and at a 64-row one
@pytest.mark.parametrize("rows,cols,m", [(128, 256, 128), (256, 512, 5), (1000, 4096, 130), (6144, 4096, 512), (4096, 14336, 64),
                                         (4096, 4096, 512), (28672, 4096, 96)])
def test_matmul_f32_rounds_no_operand(ops, rows, cols, m):
    mat, deq = q4k(ops, rows, cols, rows + cols + m)
    rng = np.random.default_rng(m)
    x = rng.normal(0, 1, (m, cols)).astype(np.float32)
    want = x.astype(np.float64) @ deq.astype(np.float64).T
    y = mat.matmul_f32(x)
    scale = float(want.std())
    err = np.abs(y - want)
    # fp32 accumulation of exact products of 22-bit activations: a few 1e-7 relative (the fp16 kernels are at 3e-4)
    assert err.max() <= 4e-6 * scale and np.sqrt((err ** 2).mean()) <= 1e-6 * scale, (err.max(), scale)
    assert np.array_equal(mat.matmul_f32(x).view(np.uint32), y.view(np.uint32))      # deterministic, also with K split over the grid
    res = rng.normal(0, 1, (m, rows)).astype(np.float32)
    assert np.abs(mat.matmul_f32(x, res) - (want + res)).max() <= 4e-6 * scale + 1e-6
    # the oracle's own fp32 product (the reference's arithmetic) is no closer to the float64 one than this
    o32 = np.stack([orc.matvec(deq, x[i]) for i in range(min(m, 4))])
    assert np.abs(y[:len(o32)] - o32).max() <= 6e-6 * scale
    mat.close()


def test_matmul_f32_reads_single_weights_and_small_activations_back(ops):
    """One-hot rows return columns of the dequantised matrix (every slot of a sub-block, both nibble halves, first and last
    super-block); activations far below one keep their low part (it is scaled before it becomes fp16)."""
    rows, cols = 384, 1024
    mat, deq = q4k(ops, rows, cols, 3)
    picks = [0, 1, 15, 16, 31, 32, 63, 64, 255, 256, 511, 777, cols - 1]
    x = np.zeros((len(picks), cols), np.float32)
    for i, j in enumerate(picks):
        x[i, j] = 1.0
    y = mat.matmul_f32(x)
    for i, j in enumerate(picks):
        assert np.abs(y[i] - deq[:, j]).max() <= 1e-7 * max(1.0, float(np.abs(deq[:, j]).max())) + 1e-8, j
    tiny = (np.random.default_rng(5).normal(0, 1, (7, cols)) * 1e-4).astype(np.float32)
    want = tiny.astype(np.float64) @ deq.astype(np.float64).T
    got = mat.matmul_f32(tiny)
    assert np.abs(got - want).max() <= 4e-6 * float(want.std())
    # linear in the activations: f(a + b) = f(a) + f(b) to fp32 rounding
    a = np.random.default_rng(6).normal(0, 1, (9, cols)).astype(np.float32)
    b = np.random.default_rng(7).normal(0, 1, (9, cols)).astype(np.float32)
    lhs, rhs = mat.matmul_f32(a + b), mat.matmul_f32(a) + mat.matmul_f32(b)
    assert np.abs(lhs - rhs).max() <= 1e-5 * float(np.abs(rhs).max())
    mat.close()


# (weight rows = 2 x feed-forward units, columns, activation rows, does the launch share K ranges between workgroups on a chip of 256
# compute units): the 8B gate|up at a full 512-row block (448 output tiles: 112 K tiles per workgroup, 1.75 output tiles) and at 384
# rows (84 K tiles), a 16-K-tile matrix (28 per workgroup), 320 output tiles of 32 K tiles (40 per workgroup), and shapes the
# plain grid keeps (fewer output tiles than compute units; a whole number of rounds; ragged rows)
SWIGLU_SHAPES = [(28672, 4096, 512, True), (28672, 4096, 384, True), (28672, 1024, 512, True), (10240, 2048, 1024, True),
                 (28672, 4096, 256, False), (16384, 1024, 512, False), (1000, 512, 130, False)]


@pytest.mark.parametrize("rows,cols,m,shared", SWIGLU_SHAPES)
def test_swiglu_epilogue_with_and_without_shared_k_ranges(ops, rows, cols, m, shared):
    """SiLU(gate) * up in the exact GEMM's epilogue against float64, with the workgroups sharing output tiles' K ranges (mode 1), on
    the plain grid (mode 0), and with every finishing workgroup computing the rest of its tile itself instead of taking its
    successor's totals (mode 2: the path a wait that runs out takes).  Mode 2 adds in the plain grid's order: bit-identical to mode 0."""
    mat, deq = q4k(ops, rows, cols, rows + cols + m)
    x = np.random.default_rng(m + 1).normal(0, 1, (m, cols)).astype(np.float32)
    y = x.astype(np.float64) @ deq.astype(np.float64).T
    gate, up = y[:, 0::2], y[:, 1::2]
    want = gate / (1.0 + np.exp(-gate)) * up
    scale, ystd = float(want.std()), float(y.std())
    got = {}
    try:
        for mode in (0, 1, 2, 1):
            ops.set_tuning("split_gemm_shared_k", mode)
            act = mat.matmul_f32_swiglu(x)
            err = np.abs(act - want)
            print(f"{rows}x{cols}, {m} rows, mode {mode}: max {err.max():.2e} rms {np.sqrt((err ** 2).mean()):.2e} (scale {scale:.3f})", flush=True)
            # gate and up carry the product's few 1e-6 (relative to its spread); d(SiLU(g) u) = SiLU'(g) u dg + SiLU(g) du
            assert (err <= 5e-6 * ystd * (np.abs(up) + np.abs(gate) + 1.0)).all() and np.sqrt((err ** 2).mean()) <= 1.5e-6 * scale, (mode, err.max(), scale)
            if mode in got:
                assert np.array_equal(got[mode].view(np.uint32), act.view(np.uint32)), mode    # deterministic across launches
            got[mode] = act
    finally:
        ops.set_tuning("split_gemm_shared_k", 1)
    assert np.array_equal(got[0].view(np.uint32), got[2].view(np.uint32))
    same = np.array_equal(got[0].view(np.uint32), got[1].view(np.uint32))
    if ops.device_info()["compute_units"] == 256:
        assert same != shared, "shared K ranges add an output tile's two parts in another order; the plain grid does not"
    mat.close()


def test_matmul_f32_refuses_other_formats(ops):
    w = np.random.default_rng(1).normal(0, 0.02, (64, 256)).astype(np.float32)
    mat = ops.Matrix(orc.FMT_Q8_0, orc.quantize(orc.FMT_Q8_0, w), 64, 256)
    with pytest.raises(Exception):
        mat.matmul_f32(np.zeros((4, 256), np.float32))
    mat.close()
