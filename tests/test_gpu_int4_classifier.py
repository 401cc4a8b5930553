"""INT4 output head on the GPU against the oracle's restatement of INT4Classifier / TensorBufferINT4: the packing
is integer work and must be identical; logits differ only by the order of fp32 sums."""
import numpy as np
import pytest

from oracle import oracle as orc

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ops():
    import espresso_amd.ops as o
    o.init()
    return o


@pytest.mark.parametrize("rows,cols", [(100, 32), (5, 7), (20, 16), (1000, 768), (32000, 768), (333, 1001)])
def test_int4_classifier_matches_oracle(ops, rows, cols):
    rng = np.random.default_rng(rows + cols)
    w = rng.normal(0, 0.02, (rows, cols)).astype(np.float32)
    w[rows // 2] += 0.05                                   # a row that wins clearly for a positive input
    if rows > 3:
        w[3] = 0.25                                        # constant row: scale 1.0, bias = the constant
    x = np.abs(rng.normal(0, 1, cols)).astype(np.float32)
    clf = ops.Int4Classifier(w)
    packed, scales, biases = clf.export()
    op, os_, ob = orc.int4_quantize(w)
    assert np.array_equal(packed, op) and np.array_equal(scales.view(np.uint32), os_.view(np.uint32))
    assert np.array_equal(biases.view(np.uint32), ob.view(np.uint32))
    logits, idx = clf.matvec_argmax(x)
    want = orc.int4_matvec(op, os_, ob, x, cols)
    tol = 1e-5 * (np.abs(want).max() + np.abs(ob).max() * np.abs(x).sum())
    assert np.abs(logits - want).max() <= tol, np.abs(logits - want).max()
    top = np.sort(want)[-2:]
    if top[1] - top[0] > 4 * tol:
        assert idx == orc.int4_argmax(op, os_, ob, x, cols)
    assert idx == int(np.argmax(logits))                   # first maximum of the GPU's own logits
    clf.close()


def test_int4_reference_cases(ops):
    """Tests/EspressoTests/INT4ClassifierTests.swift:8-71 (row 73) and :144-173 (odd dimension, row 3)."""
    w = np.zeros((100, 32), np.float32)
    for r in range(100):
        w[r] = np.float32(r) * np.float32(0.01) + np.arange(32, dtype=np.float32) * np.float32(0.001)
    w[73] = 10.0
    assert ops.Int4Classifier(w).matvec_argmax(np.ones(32, np.float32))[1] == 73
    w = np.full((5, 7), 0.5, np.float32)
    w[3] = 10.0
    assert ops.Int4Classifier(w).matvec_argmax(np.ones(7, np.float32))[1] == 3
    # ties: the lowest index wins
    w = np.tile(np.linspace(-1, 1, 16, dtype=np.float32), (6, 1))
    assert ops.Int4Classifier(w).matvec_argmax(np.ones(16, np.float32))[1] == 0
