"""The Q8_0 GEMV on the matrix cores (768, 2048 and 4096 columns, one and two activation rows) against the oracle's matvec on the
dequantised weights and against the dot-product kernel, stand-alone and inside the 6-layer model's decoder."""
import numpy as np
import pytest

from oracle import oracle as orc

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def mods():
    import espresso_amd.llama as ll
    import espresso_amd.ops as ops
    import espresso_amd.synthetic as syn
    ops.init()
    yield ll, ops, syn
    ops.set_tuning("q80_mfma", -1)


def q80_matrix(ops, rows, cols, seed):
    w = np.random.default_rng(seed).normal(0, 0.02, (rows, cols)).astype(np.float32)
    blocks = orc.quantize(orc.FMT_Q8_0, w)
    return ops.Matrix(orc.FMT_Q8_0, blocks, rows, cols), orc.dequantize(orc.FMT_Q8_0, blocks, rows * cols).reshape(rows, cols)


# BASELINE configs[1]'s isolated shapes (768 x 768, 2048 x 768, 768 x 2048, 32000 x 768), ragged and tall ones, 4096 columns
@pytest.mark.parametrize("rows,cols", [(768, 768), (2048, 768), (768, 2048), (32000, 768), (1000, 768), (30, 2048), (4096, 4096), (20000, 4096)])
def test_matches_oracle_and_dot_product_kernel(mods, rows, cols):
    ll, ops, syn = mods
    mat, deq = q80_matrix(ops, rows, cols, rows + cols)
    assert mat.resident_bytes > mat.bytes            # the tiled copy exists
    rng = np.random.default_rng(rows)
    scale = np.abs(deq).max() * np.sqrt(cols)
    for batch in (1, 2, 3):
        x = rng.normal(0, 1, (batch, cols)).astype(np.float16)
        res = rng.normal(0, 1, (batch, rows)).astype(np.float32)
        want = np.stack([orc.matvec(deq, x[b].astype(np.float32)) for b in range(batch)])
        ops.set_tuning("q80_mfma", 0)
        base = mat.gemv(x)
        ops.set_tuning("q80_mfma", 1)
        y = mat.gemv(x)
        tol = (2e-5 if batch <= 2 else 1e-3) * scale + 1e-6      # three rows: a pair and a single, or the fp16-weight GEMM
        assert np.abs(y - want).max() <= tol, (batch, float(np.abs(y - want).max()), scale)
        assert np.abs(y - base).max() <= tol
        assert np.array_equal(mat.gemv(x).view(np.uint32), y.view(np.uint32))
        assert np.abs(mat.gemv(x, res) - (want + res)).max() <= tol + 1e-5
    ops.set_tuning("q80_mfma", 1)
    for j in (0, 7, 8, 15, 16, 31, 32, 255, 256, cols - 1):
        x = np.zeros((2, cols), np.float16)
        x[0, j] = 1.0; x[1, cols - 1 - j] = -2.0
        y = mat.gemv(x)
        assert np.abs(y[0] - deq[:, j]).max() <= 1e-6 * max(1.0, float(np.abs(deq[:, j]).max())) + 1e-7, j
        assert np.abs(y[1] + 2.0 * deq[:, cols - 1 - j]).max() <= 2e-6 * max(1.0, float(np.abs(deq[:, j]).max())) + 1e-7, j
    ops.set_tuning("q80_mfma", -1)
    mat.close()


def test_stories_shape_decoder_on_the_matrix_cores(mods):
    """Two layers of the 6-layer model's shape, Q8_0: fused-norm staging, RoPE / KV write, merged attention in wo, SwiGLU and the
    32000-row head with its arg-max epilogue, against the oracle; the stream equals the dot-product kernels' and the two-token loop's."""
    import model_util as mu
    ll, ops, syn = mods
    kw = dict(n_layer=2, n_head=12, n_kv_head=12, d_model=768, head_dim=64, hidden_dim=2048, vocab=32000, max_seq=96)
    ocfg = orc.LlamaConfig(gemv_inputs_fp16=True, **kw)
    packed, deq = mu.pack_weights(mu.random_weights(ocfg, 5, std=0.02), orc.FMT_Q8_0)
    o = mu.load_oracle(ocfg, deq)

    def build():
        g = ll.LlamaRuntime(ll.MultiModelConfig(**kw))
        ll.load_packed_weights(g, packed, orc.FMT_Q8_0)
        return g
    ops.set_tuning("q80_mfma", 1)      # every GEMV of the step on the matrix cores
    g = build()
    prompt = np.random.default_rng(2).integers(0, 32000, 12).tolist()
    o.prefill(prompt); g.prefill(prompt)
    for step in range(6):
        assert np.abs(o.last_hidden() - g.last_hidden()).max() <= 2e-3 * max(1.0, float(np.abs(o.last_hidden()).max()))
        assert np.abs(o.logits() - g.logits()).max() <= 2e-2
        tok = o.select_greedy()
        if o.top2_margin() > 1e-3:
            assert g.select_greedy() == tok
        o.advance(tok); g.advance(tok)
    plain = g.generate(prompt, 40)[0]
    twin = build()
    assert ll.generate_two_token(g, twin, prompt, 40)[0] == plain
    ops.set_tuning("q80_mfma", 0)
    ref = build()
    want, margin = o.generate(prompt, 40, with_margin=True)
    if margin > 1e-3:
        assert ref.generate(prompt, 40)[0] == want and plain == want
    ops.set_tuning("q80_mfma", -1)
    for r in (g, twin, ref):
        r.close()


# the same kernel with fp16 weights as its B operand (BASELINE configs[0] and [4]: the 6-layer model with fp16 weights)
@pytest.mark.parametrize("rows,cols", [(768, 768), (2048, 768), (768, 2048), (32000, 768), (1000, 768), (30, 2048)])
def test_fp16_weights_on_the_matrix_cores(mods, rows, cols):
    ll, ops, syn = mods
    w = np.random.default_rng(rows + cols).normal(0, 0.02, (rows, cols)).astype(np.float32)
    blocks = orc.quantize(orc.FMT_F16, w)
    deq = orc.dequantize(orc.FMT_F16, blocks, rows * cols).reshape(rows, cols)
    mat = ops.Matrix(orc.FMT_F16, blocks, rows, cols)
    assert mat.resident_bytes > mat.bytes
    rng = np.random.default_rng(cols)
    scale = np.abs(deq).max() * np.sqrt(cols)
    for batch in (1, 2):
        x = rng.normal(0, 1, (batch, cols)).astype(np.float16)
        res = rng.normal(0, 1, (batch, rows)).astype(np.float32)
        want = np.stack([orc.matvec(deq, x[b].astype(np.float32)) for b in range(batch)])
        ops.set_tuning("q80_mfma", 0)
        base = mat.gemv(x)
        ops.set_tuning("q80_mfma", 1)
        y = mat.gemv(x)
        assert np.abs(y - want).max() <= 2e-6 * scale + 1e-6, (batch, float(np.abs(y - want).max()))   # exact products, fp32 sums
        assert np.abs(y - base).max() <= 2e-6 * scale + 1e-6
        assert np.array_equal(mat.gemv(x).view(np.uint32), y.view(np.uint32))
        assert np.abs(mat.gemv(x, res) - (want + res)).max() <= 2e-6 * scale + 1e-5
    for j in (0, 1, 2, 3, 7, 8, 31, 32, 255, 256, cols - 1):
        x = np.zeros((2, cols), np.float16)
        x[0, j] = 1.0; x[1, cols - 1 - j] = -2.0
        y = mat.gemv(x)
        assert np.array_equal(y[0], deq[:, j]), j
        assert np.array_equal(y[1], -2.0 * deq[:, cols - 1 - j]), j
    ops.set_tuning("q80_mfma", -1)
    mat.close()
