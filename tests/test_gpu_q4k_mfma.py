"""The Q4_K GEMV that runs on the matrix cores (one to eight activation rows per pass over the weights), against the
oracle's matvec on the dequantised weights and against the dot-product kernels, stand-alone and inside the decoder."""
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
    ops.set_tuning("q4k_mfma", -1)
    ops.set_tuning("q4k_mfma_waves", 0)
    ops.set_tuning("q4k_mfma_ks", 0)
    ops.set_tuning("q4k_wide", 1)


def q4k_matrix(ops, rows, cols, seed):
    w = np.random.default_rng(seed).normal(0, 0.02, (rows, cols)).astype(np.float32)
    blocks = orc.quantize(orc.FMT_Q4_K, w)
    return ops.Matrix(orc.FMT_Q4_K, blocks, rows, cols), orc.dequantize(orc.FMT_Q4_K, blocks, rows * cols).reshape(rows, cols)


@pytest.mark.parametrize("rows,cols", [(16, 4096), (1000, 4096), (4096, 4096), (6144, 4096), (28672, 4096), (130, 14336), (4096, 14336)])
def test_matches_oracle_and_dot_product_kernels(mods, rows, cols):
    ll, ops, syn = mods
    mat, deq = q4k_matrix(ops, rows, cols, rows + cols)
    rng = np.random.default_rng(rows)
    scale = np.abs(deq).max() * np.sqrt(cols)
    for batch in (1, 2, 3, 4, 7, 8):
        x = rng.normal(0, 1, (batch, cols)).astype(np.float16)
        res = rng.normal(0, 1, (batch, rows)).astype(np.float32)
        want = np.stack([orc.matvec(deq, x[b].astype(np.float32)) for b in range(batch)])
        ops.set_tuning("q4k_mfma", 0)
        base = mat.gemv(x) if batch <= 2 else None
        for waves, ks in (((0, 0), (4, 1), (8, 8), (16, 16)) if cols == 4096 else ((0, 0), (4, 4), (8, 8), (16, 8))):
            ops.set_tuning("q4k_mfma", 1)
            ops.set_tuning("q4k_mfma_waves", waves)
            ops.set_tuning("q4k_mfma_ks", ks)
            y = mat.gemv(x)
            # exact products, fp32 sums: only the order of additions differs from the oracle's
            assert np.abs(y - want).max() <= 2e-5 * scale + 1e-6, (batch, ks, np.abs(y - want).max())
            if base is not None:
                assert np.abs(y - base).max() <= 2e-5 * scale + 1e-6
            assert np.array_equal(mat.gemv(x).view(np.uint32), y.view(np.uint32))      # deterministic
            yr = mat.gemv(x, res)
            assert np.abs(yr - (want + res)).max() <= 2e-5 * scale + 1e-5
    # one-hot activations read columns of the dequantised matrix back, in every slot of a four-row pass
    ops.set_tuning("q4k_mfma", 1)
    ops.set_tuning("q4k_mfma_waves", 0)
    ops.set_tuning("q4k_mfma_ks", 0)
    for j in (0, 7, 31, 32, 255, 256, cols - 1):
        x = np.zeros((4, cols), np.float16)
        x[0, j] = 1.0; x[1, (j + 1) % cols] = 1.0; x[2, (j + 33) % cols] = 2.0; x[3, cols - 1 - j] = -1.0
        y = mat.gemv(x)
        for b, (col, f) in enumerate([(j, 1.0), ((j + 1) % cols, 1.0), ((j + 33) % cols, 2.0), (cols - 1 - j, -1.0)]):
            assert np.abs(y[b] - f * deq[:, col]).max() <= 1e-6 * max(1.0, np.abs(deq[:, col]).max()) + 1e-7, (j, b)
    mat.close()


@pytest.mark.parametrize("rows,cols", [(16, 4096), (1000, 4096), (14336, 4096), (28672, 4096), (130, 14336), (4096, 14336),
                                       (2048, 1024), (100, 2048), (3072, 3072), (2050, 8192)])
def test_five_to_eight_rows_in_one_pass(mods, rows, cols):
    """Five to eight activation rows on the kernel that folds the sub-block scales into the B operand (exact integer sc * q, a second
    MFMA chain for the minimums), activations staged per workgroup or per wavefront tile: against the oracle's matvec, against the
    nibble-B GEMM kernel it replaces, residual form, determinism, one-hot columns in every row."""
    ll, ops, syn = mods
    for key, value in (("q4k_mfma", -1), ("q4k_mfma_waves", 0), ("q4k_mfma_ks", 0)):
        ops.set_tuning(key, value)
    mat, deq = q4k_matrix(ops, rows, cols, rows + cols + 1)
    rng = np.random.default_rng(rows + 5)
    scale = np.abs(deq).max() * np.sqrt(cols)
    for batch in (5, 6, 7, 8):
        x = rng.normal(0, 1, (batch, cols)).astype(np.float16)
        res = rng.normal(0, 1, (batch, rows)).astype(np.float32)
        want = x.astype(np.float64) @ deq.astype(np.float64).T
        ops.set_tuning("q4k_wide", 0)
        base = mat.gemv(x)
        assert np.abs(base - want).max() <= 2e-5 * scale + 1e-6
        for form in ((1, 2, 3) if cols == 4096 else (1,)):
            ops.set_tuning("q4k_wide", form)
            y = mat.gemv(x)
            # exact products, fp32 sums over 256 columns at a time inside the matrix core
            assert np.abs(y - want).max() <= 2e-6 * scale + 1e-6, (batch, form, np.abs(y - want).max() / scale)
            assert np.array_equal(mat.gemv(x).view(np.uint32), y.view(np.uint32))
            assert np.abs(mat.gemv(x, res) - (want + res)).max() <= 2e-6 * scale + 1e-5
    ops.set_tuning("q4k_wide", 1)
    for j in (0, 7, 31, 32, 63, 64, 255, 256, cols - 1):
        x = np.zeros((8, cols), np.float16)
        picks = [(j + 37 * b) % cols for b in range(8)]
        for b, c in enumerate(picks):
            x[b, c] = 1.0 + b
        y = mat.gemv(x)
        for b, c in enumerate(picks):
            assert np.abs(y[b] - (1.0 + b) * deq[:, c]).max() <= 1e-6 * (1.0 + b) * max(1.0, np.abs(deq[:, c]).max()) + 1e-7, (j, b)
    mat.close()


# the other widths of the reference's model registry (ModelRegistry.swift:59-107): llama3.2-1B d 2048 / FFN 8192, llama3.2-3B d 3072,
# Qwen3-0.6B d 1024 / FFN 3072; ragged row counts included
@pytest.mark.parametrize("rows,cols", [(2048, 1024), (1000, 1024), (6144, 1024), (2048, 2048), (16384, 2048), (3072, 3072), (1024, 3072),
                                       (2048, 8192), (3072, 8192), (40, 8192)])
def test_registry_widths_on_the_matrix_cores(mods, rows, cols):
    ll, ops, syn = mods
    mat, deq = q4k_matrix(ops, rows, cols, rows + cols)
    assert mat.resident_bytes > mat.bytes            # the tiled copy exists: these widths run on the matrix cores
    rng = np.random.default_rng(rows + 1)
    scale = np.abs(deq).max() * np.sqrt(cols)
    for batch in (1, 2):
        x = rng.normal(0, 1, (batch, cols)).astype(np.float16)
        res = rng.normal(0, 1, (batch, rows)).astype(np.float32)
        want = np.stack([orc.matvec(deq, x[b].astype(np.float32)) for b in range(batch)])
        ops.set_tuning("q4k_mfma", 0)
        base = mat.gemv(x)
        ops.set_tuning("q4k_mfma", -1)
        y = mat.gemv(x)
        assert np.abs(y - want).max() <= 2e-5 * scale + 1e-6, (batch, np.abs(y - want).max())
        assert np.abs(y - base).max() <= 2e-5 * scale + 1e-6
        assert np.array_equal(mat.gemv(x).view(np.uint32), y.view(np.uint32))
        assert np.abs(mat.gemv(x, res) - (want + res)).max() <= 2e-5 * scale + 1e-5
    for j in (0, 31, 255, 256, cols - 1):
        x = np.zeros((2, cols), np.float16)
        x[0, j] = 1.0; x[1, cols - 1 - j] = -2.0
        y = mat.gemv(x)
        assert np.abs(y[0] - deq[:, j]).max() <= 1e-6 * max(1.0, np.abs(deq[:, j]).max()) + 1e-7
        assert np.abs(y[1] + 2.0 * deq[:, cols - 1 - j]).max() <= 2e-6 * max(1.0, np.abs(deq[:, j]).max()) + 1e-7
    mat.close()


@pytest.mark.parametrize("name,shape", [
    ("llama3.2-1b width", dict(n_head=32, n_kv_head=8, d_model=2048, head_dim=64, hidden_dim=8192)),
    ("llama3.2-3b width", dict(n_head=24, n_kv_head=8, d_model=3072, head_dim=128, hidden_dim=8192)),
    ("qwen3-0.6b width", dict(n_head=16, n_kv_head=8, d_model=1024, head_dim=128, hidden_dim=3072)),
])
def test_registry_width_decoders_match_oracle(mods, name, shape):
    """Two layers at each registry width, Q4_K, fp16 KV: fused-norm, merge and SwiGLU forms of the matrix-core GEMV with split
    activations against the oracle in the reference's default arithmetic, then graph replay against the eager steps."""
    from test_gpu_full_size import oracle_from_packed
    ll, ops, syn = mods
    cfg = ll.MultiModelConfig(**dict(shape, n_layer=2, vocab=4096, max_seq=64, norm_eps=1e-5, rope_theta=500000.0, name=name))
    g, packed = syn.build_runtime(cfg, orc.FMT_Q4_K, seed=31, kv_format=orc.FMT_F16, keep_packed=True)
    assert g.resident_weight_bytes > g.weight_bytes
    o = oracle_from_packed(cfg, packed, orc.FMT_Q4_K, 2, True, 64, gemv_inputs_fp16=False)
    prompt = [1, 4000, 777, 2048, 5, 902, 3133, 2]
    o.prefill(prompt)
    g.prefill(np.asarray(prompt, np.uint32))
    worst = 0.0
    for step in range(6):
        ho, hg = o.last_hidden(), g.last_hidden()
        assert np.abs(ho - hg).max() <= 1e-3 * max(1.0, np.abs(ho).max())
        worst = max(worst, float(np.abs(o.logits() - g.logits()).max()))
        tok = o.select_greedy()
        if o.top2_margin() > 1e-3:
            assert g.select_greedy() == tok
        o.advance(tok); g.advance(tok)
    print(f"{name}: worst logit difference over 6 steps {worst:.3e}")
    assert worst <= 2e-3
    plain = g.generate(prompt, 20)[0]
    ll.set_graph_replay(g, False)
    assert g.generate(prompt, 20)[0] == plain
    g.close()


@pytest.mark.parametrize("waves,ks", [(0, 0), (4, 1), (16, 16)])
def test_decoder_with_matrix_core_gemvs_matches_oracle(mods, waves, ks):
    """One layer of the 8B shape: fused RMSNorm staging, RoPE / KV-write, SwiGLU and residual epilogues, attention states merged
    in the wo GEMV - all through the matrix-core kernel - against the oracle, then the two-row verify step."""
    from test_gpu_full_size import oracle_from_packed
    ll, ops, syn = mods
    ops.set_tuning("q4k_mfma", 1)
    ops.set_tuning("q4k_mfma_waves", waves)
    ops.set_tuning("q4k_mfma_ks", ks)
    cfg = ll.MultiModelConfig(**dict(syn.LLAMA3_8B, n_layer=1, max_seq=48))
    g, packed = syn.build_runtime(cfg, orc.FMT_Q4_K, seed=9, kv_format=orc.FMT_F16, keep_packed=True)
    o = oracle_from_packed(cfg, packed, orc.FMT_Q4_K, 1, True, 48)
    prompt = [1, 128255, 777, 64000, 5, 90210, 31337, 2]
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
    # graph replay and the two-token loop (two-row passes) give the plain stream
    plain = g.generate(prompt, 24)[0]
    ops.set_tuning("q4k_mfma", 0)
    reference_kernels = syn.build_runtime(cfg, orc.FMT_Q4_K, seed=9, kv_format=orc.FMT_F16)[0]
    want = reference_kernels.generate(prompt, 24)[0]
    ops.set_tuning("q4k_mfma", 1)
    twin = syn.build_runtime(cfg, orc.FMT_Q4_K, seed=9, kv_format=orc.FMT_F16)[0]
    got, st = ll.generate_two_token(g, twin, prompt, 24)
    assert got == plain
    margin_ok = o.generate(prompt, 24, with_margin=True)[1] > 1e-3
    if margin_ok:
        assert plain == want
    for r in (g, twin, reference_kernels):
        r.close()
