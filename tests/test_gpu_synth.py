"""GPU: seeded synthetic weights are deterministic, valid blocks, and N(0, std) distributed."""
import numpy as np
import pytest

from oracle import oracle as orc

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ops():
    import espresso_amd.ops as o
    o.init()
    return o


@pytest.mark.parametrize("fmt", [orc.FMT_F16, orc.FMT_Q8_0, orc.FMT_Q4_0, orc.FMT_Q4_K])
def test_synth_weights(ops, fmt):
    n = 256 * 2048
    a = ops.synth_weights(fmt, 7, 0.02, n)
    assert np.array_equal(a, ops.synth_weights(fmt, 7, 0.02, n))
    assert not np.array_equal(a, ops.synth_weights(fmt, 8, 0.02, n))
    # a longer stream starts with the same elements (value depends only on seed and index)
    assert np.array_equal(a, ops.synth_weights(fmt, 7, 0.02, 2 * n)[:a.size])
    w = orc.dequantize(fmt, a, n)
    assert np.all(np.isfinite(w))
    assert abs(w.mean()) < 2e-4 and abs(w.std() - 0.02) < 1.5e-3
    assert 0.06 < np.abs(w).max() < 0.12
    if fmt == orc.FMT_Q8_0:      # absmax quantisation: every block reaches +-127
        q = a.reshape(-1, 34)[:, 2:].view(np.int8)
        assert np.all(np.abs(q).max(axis=1) == 127)
        ref = orc.dequantize(orc.FMT_F16, ops.synth_weights(orc.FMT_F16, 7, 0.02, n), n)
        assert np.abs(w - ref).max() < 0.12 / 127 * 0.51 + 1e-4   # within half a step of the (fp16-rounded) draw
    if fmt == orc.FMT_Q4_0:      # the largest-magnitude element sits at nibble 0 (= -8 d)
        qs = a.reshape(-1, 18)[:, 2:]
        nib = np.concatenate([qs & 0xF, qs >> 4], axis=1)
        assert np.all(nib.min(axis=1) == 0)
    if fmt == orc.FMT_Q4_K:      # 6-bit scales and mins both reach 63 in every super-block
        import numpy_ref as ref
        sc, m = ref.q4_k_scales_mins(a.reshape(-1, 144)[:, 4:16])
        assert np.all(sc.max(axis=1) == 63) and np.all(m.max(axis=1) == 63)
        draws = orc.dequantize(orc.FMT_F16, ops.synth_weights(orc.FMT_F16, 7, 0.02, n), n)
        assert np.linalg.norm(w - draws) / np.linalg.norm(draws) < 0.12
