"""The Q4_0 GEMV that runs on the matrix cores (one to four activation rows per pass over a tiled copy of the nibble and scale
planes), against the oracle's matvec on the dequantised weights and against the dot-product kernel, stand-alone and inside
the decoder."""
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
    for key, value in (("q40_mfma", -1), ("q4k_mfma_waves", 0), ("q4k_mfma_ks", 0), ("q4k_wide", 1)):
        ops.set_tuning(key, value)


def q40_matrix(ops, rows, cols, seed):
    w = np.random.default_rng(seed).normal(0, 0.02, (rows, cols)).astype(np.float32)
    blocks = orc.quantize(orc.FMT_Q4_0, w)
    return ops.Matrix(orc.FMT_Q4_0, blocks, rows, cols), orc.dequantize(orc.FMT_Q4_0, blocks, rows * cols).reshape(rows, cols)


@pytest.mark.parametrize("rows,cols", [(16, 4096), (1000, 4096), (4096, 4096), (14336, 4096), (32000, 4096), (130, 14336), (4096, 14336)])
def test_matches_oracle_and_dot_product_kernel(mods, rows, cols):
    ll, ops, syn = mods
    mat, deq = q40_matrix(ops, rows, cols, rows + cols)
    rng = np.random.default_rng(rows)
    scale = np.abs(deq).max() * np.sqrt(cols)
    variants = ((0, 0), (4, 2), (8, 4), (8, 8)) if cols == 4096 else ((0, 0), (7, 7), (14, 14), (14, 7), (8, 4))
    for batch in (1, 2, 3, 4, 5, 8):
        x = rng.normal(0, 1, (batch, cols)).astype(np.float16)
        res = rng.normal(0, 1, (batch, rows)).astype(np.float32)
        want = np.stack([orc.matvec(deq, x[b].astype(np.float32)) for b in range(batch)])
        ops.set_tuning("q40_mfma", 0)
        base = mat.gemv(x)
        assert np.abs(base - want).max() <= 3e-4 * scale + 1e-6      # the dot-product kernel rounds d (n - 8) to fp16 first
        for waves, ks in variants:
            ops.set_tuning("q40_mfma", 1)
            ops.set_tuning("q4k_mfma_waves", waves)
            ops.set_tuning("q4k_mfma_ks", ks)
            y = mat.gemv(x)
            # exact products, fp32 sums: only the order of additions differs from the oracle's (five rows and more of the larger
            # matrices take the MFMA GEMM kernels, whose weights are d (n - 8) rounded to fp16)
            tol = (2e-5 if batch <= 4 or (cols == 4096 and rows <= 8192) else 3e-4) * scale
            assert np.abs(y - want).max() <= tol + 1e-6, (batch, waves, ks, float(np.abs(y - want).max()), scale)
            assert np.array_equal(mat.gemv(x).view(np.uint32), y.view(np.uint32))      # deterministic
            yr = mat.gemv(x, res)
            assert np.abs(yr - (want + res)).max() <= tol + 1e-5
    # one-hot activations read columns of the dequantised matrix back, in every slot of a four-row pass
    ops.set_tuning("q40_mfma", 1)
    ops.set_tuning("q4k_mfma_waves", 0)
    ops.set_tuning("q4k_mfma_ks", 0)
    for j in (0, 7, 15, 16, 31, 32, 511, 512, cols - 1):
        x = np.zeros((4, cols), np.float16)
        picks = [(j, 1.0), ((j + 1) % cols, 1.0), ((j + 33) % cols, 2.0), (cols - 1 - j, -1.0)]
        for b, (col, f) in enumerate(picks):
            x[b, col] = f
        y = mat.gemv(x)
        for b, (col, f) in enumerate(picks):
            assert np.abs(y[b] - f * deq[:, col]).max() <= 1e-6 * max(1.0, np.abs(deq[:, col]).max()) + 1e-7, (j, b)
    mat.close()


@pytest.mark.parametrize("mode", [1, -1])
def test_decoder_with_matrix_core_q4_0_gemvs_matches_oracle(mods, mode):
    """One layer of the 8B shape in Q4_0 through the matrix-core kernel (fused RMSNorm staging, RoPE / KV-write, SwiGLU and residual
    epilogues, attention states merged in the wo GEMV, arg-max head) against the oracle, then the two-row verify step."""
    from test_gpu_full_size import oracle_from_packed
    ll, ops, syn = mods
    ops.set_tuning("q40_mfma", mode)
    cfg = ll.MultiModelConfig(**dict(syn.LLAMA3_8B, n_layer=1, max_seq=48, vocab=32000))
    g, packed = syn.build_runtime(cfg, orc.FMT_Q4_0, seed=9, kv_format=orc.FMT_F16, keep_packed=True)
    o = oracle_from_packed(cfg, packed, orc.FMT_Q4_0, 1, True, 48)
    prompt = [1, 31999, 777, 16000, 5, 9021, 31337, 2]
    o.prefill(prompt)
    g.prefill(np.asarray(prompt, np.uint32))
    for step in range(5):
        ho, hg = o.last_hidden(), g.last_hidden()
        assert np.abs(ho - hg).max() <= 2e-3 * max(1.0, np.abs(ho).max())
        assert np.abs(o.logits() - g.logits()).max() <= 2e-2
        tok = o.select_greedy()
        if o.top2_margin() > 1e-3:
            assert g.select_greedy() == tok
        o.advance(tok); g.advance(tok)
    plain = g.generate(prompt, 24)[0]
    twin = syn.build_runtime(cfg, orc.FMT_Q4_0, seed=9, kv_format=orc.FMT_F16)[0]
    got, st = ll.generate_two_token(g, twin, prompt, 24)
    assert got == plain
    ops.set_tuning("q40_mfma", 0)
    reference_kernels = syn.build_runtime(cfg, orc.FMT_Q4_0, seed=9, kv_format=orc.FMT_F16)[0]
    want = reference_kernels.generate(prompt, 24)[0]
    if o.generate(prompt, 24, with_margin=True)[1] > 1e-3:
        assert plain == want
    for r in (g, twin, reference_kernels):
        r.close()


@pytest.mark.parametrize("rows,cols", [(16, 4096), (1000, 4096), (14336, 4096), (28672, 4096), (130, 14336), (4096, 14336)])
def test_five_to_eight_rows_in_one_pass(mods, rows, cols):
    """Five to eight activation rows on the kernel whose every MFMA contracts one 32-weight block for sixteen weight rows (B = the exact
    integer q - 8, the block's scale applied to the accumulator): against the oracle's matvec and the kernels it replaces, both ways of
    staging the activations, residual form, determinism, one-hot columns in every row."""
    ll, ops, syn = mods
    for key, value in (("q40_mfma", -1), ("q4k_mfma_waves", 0), ("q4k_mfma_ks", 0)):
        ops.set_tuning(key, value)
    mat, deq = q40_matrix(ops, rows, cols, rows + cols + 1)
    rng = np.random.default_rng(rows + 5)
    scale = np.abs(deq).max() * np.sqrt(cols)
    for batch in (5, 6, 7, 8):
        x = rng.normal(0, 1, (batch, cols)).astype(np.float16)
        res = rng.normal(0, 1, (batch, rows)).astype(np.float32)
        want = x.astype(np.float64) @ deq.astype(np.float64).T
        ops.set_tuning("q4k_wide", 0)
        base = mat.gemv(x)
        assert np.abs(base - want).max() <= 3e-4 * scale + 1e-6
        for form in ((1, 2, 3) if cols == 4096 else (1,)):
            ops.set_tuning("q4k_wide", form)
            y = mat.gemv(x)
            assert np.abs(y - want).max() <= 2e-6 * scale + 1e-6, (batch, form, np.abs(y - want).max() / scale)
            assert np.array_equal(mat.gemv(x).view(np.uint32), y.view(np.uint32))
            assert np.abs(mat.gemv(x, res) - (want + res)).max() <= 2e-6 * scale + 1e-5
    ops.set_tuning("q4k_wide", 1)
    for j in (0, 3, 4, 15, 16, 31, 32, 255, 256, 511, 512, cols - 1):
        x = np.zeros((8, cols), np.float16)
        picks = [(j + 37 * b) % cols for b in range(8)]
        for b, c in enumerate(picks):
            x[b, c] = 1.0 + b
        y = mat.gemv(x)
        for b, c in enumerate(picks):
            assert np.abs(y[b] - (1.0 + b) * deq[:, c]).max() <= 1e-6 * (1.0 + b) * max(1.0, np.abs(deq[:, c]).max()) + 1e-7, (j, b)
    mat.close()
