"""GPU parity at the benchmark's full sizes: the weight-GEMV shapes of Llama-3-8B against the oracle's matvec, one
8B-shaped layer plus the 128256-row head against the oracle runtime, and the whole 32-layer model through
properties that do not need a CPU run (graph replay = eager launches, rollback and regenerate, exact two-token
stream = plain greedy, block prefill then decode = the token walk's cache)."""
import numpy as np
import pytest

from oracle import oracle as orc

pytestmark = pytest.mark.gpu

LOGIT_TOL = 2e-2


@pytest.fixture(scope="module")
def mods():
    import espresso_amd.llama as ll
    import espresso_amd.ops as ops
    import espresso_amd.synthetic as syn
    ops.init()
    return ll, ops, syn


def tiled_blocks(fmt, rows, cols, seed, period=1031):
    """Quantised rows with a period that divides no tile or team size, so a wrong row index cannot go unnoticed."""
    rng = np.random.default_rng(seed)
    base_rows = min(rows, period)
    w = rng.normal(0, 0.02, (base_rows, cols)).astype(np.float32)
    blk = orc.quantize(fmt, w)
    deq = orc.dequantize(fmt, blk, base_rows * cols).reshape(base_rows, cols)
    reps = -(-rows // base_rows)
    row_bytes = blk.size // base_rows
    blocks = np.tile(blk.reshape(base_rows, row_bytes), (reps, 1))[:rows].reshape(-1)
    return np.ascontiguousarray(blocks), np.tile(deq, (reps, 1))[:rows]


# BASELINE configs[2]: 4096x4096, 1024x4096, 14336x4096, 4096x14336 in Q4_K and Q4_0; configs[1]'s head in Q8_0
@pytest.mark.parametrize("name,rows,cols", [
    ("q4_k", 4096, 4096), ("q4_k", 1024, 4096), ("q4_k", 14336, 4096), ("q4_k", 4096, 14336), ("q4_k", 28672, 4096),
    ("q4_0", 4096, 4096), ("q4_0", 14336, 4096), ("q4_0", 4096, 14336), ("q8_0", 32000, 768),
    ("q8_0", 16390, 256),   # a tall matrix (four rows per wavefront) whose last workgroup is ragged
])
def test_full_size_weight_gemv_matches_oracle(mods, name, rows, cols):
    ll, ops, syn = mods
    fmt = {"q4_k": orc.FMT_Q4_K, "q4_0": orc.FMT_Q4_0, "q8_0": orc.FMT_Q8_0}[name]
    blocks, deq = tiled_blocks(fmt, rows, cols, seed=rows + cols)
    mat = ops.Matrix(fmt, blocks, rows, cols)
    rng = np.random.default_rng(rows * 3 + cols)
    scale = np.abs(deq).max() * np.sqrt(cols)
    for batch in (1, 2, 8):
        x = rng.normal(0, 1, (batch, cols)).astype(np.float16)
        y = mat.gemv(x)
        want = np.stack([orc.matvec(deq, x[b].astype(np.float32)) for b in range(batch)])
        # batch 1-2: fp32 sums of exact products, only the order differs; batch 8 takes the MFMA kernel, whose
        # weights are rounded to fp16 once (relative 2^-11 per weight)
        tol = 2e-5 * scale + 1e-6 if batch <= 2 else 1e-3 * scale
        assert np.abs(y - want).max() <= tol, (batch, np.abs(y - want).max(), tol)
    # a one-hot activation reads one column of the dequantised matrix back
    for j in (0, 31, 255, cols - 1):
        x = np.zeros((1, cols), np.float16)
        x[0, j] = 1.0
        y = mat.gemv(x)[0]
        assert np.abs(y - deq[:, j]).max() <= 1e-6 * max(1.0, np.abs(deq[:, j]).max()) + 1e-7
    mat.close()


oracle_from_packed = orc.runtime_from_packed


def test_8b_shaped_layer_and_head_match_oracle(mods):
    """One layer of the 8B shape (d 4096, 32/8 heads x 128, FFN 14336) and the 128256-row head, Q4_K, fp16 KV."""
    ll, ops, syn = mods
    cfg = ll.MultiModelConfig(**dict(syn.LLAMA3_8B, n_layer=1, max_seq=32))
    g, packed = syn.build_runtime(cfg, orc.FMT_Q4_K, seed=9, kv_format=orc.FMT_F16, keep_packed=True)
    o = oracle_from_packed(cfg, packed, orc.FMT_Q4_K, 1, True, 32)
    prompt = [1, 128255, 777, 64000, 5, 90210, 31337, 2]
    o.prefill(prompt)
    g.prefill(np.asarray(prompt, np.uint32))
    worst = 0.0
    for step in range(5):
        ho, hg = o.last_hidden(), g.last_hidden()
        assert np.abs(ho - hg).max() <= 2e-3 * max(1.0, np.abs(ho).max())
        lo, lg = o.logits(), g.logits()
        worst = max(worst, float(np.abs(lo - lg).max()))
        assert worst <= LOGIT_TOL
        tok = o.select_greedy()
        if o.top2_margin() > 1e-3:
            assert g.select_greedy() == tok
        o.advance(tok)
        g.advance(tok)
    print(f"8B-shaped layer + head: worst logit difference {worst:.2e}")
    g.close()

def test_8b_shaped_layer_prompt_block_matches_oracle(mods):
    """A 160-token prompt through one layer of the 8B shape: the block path at its real sizes (two row tiles of the MFMA
    GEMM, gate|up without split-K so that SwiGLU runs in the GEMM's epilogue, causal attention on the matrix cores with a
    ragged last tile) against the oracle's token-by-token walk."""
    ll, ops, syn = mods
    cfg = ll.MultiModelConfig(**dict(syn.LLAMA3_8B, n_layer=1, max_seq=176))
    g, packed = syn.build_runtime(cfg, orc.FMT_Q4_K, seed=21, kv_format=orc.FMT_F16, keep_packed=True)
    o = oracle_from_packed(cfg, packed, orc.FMT_Q4_K, 1, True, 176)
    prompt = np.random.default_rng(160).integers(0, cfg.vocab, 160).astype(np.uint32)
    o.prefill([int(t) for t in prompt])
    g.prefill(prompt)
    ho, hg = o.last_hidden(), g.last_hidden()
    assert np.abs(ho - hg).max() <= 4e-3 * max(1.0, np.abs(ho).max()), np.abs(ho - hg).max()
    assert np.abs(o.logits() - g.logits()).max() <= LOGIT_TOL
    ll.set_matrix_prefill(g, False)
    g.reset()
    g.prefill(prompt)
    assert np.abs(g.last_hidden() - hg).max() <= 4e-3 * max(1.0, np.abs(ho).max())
    g.close()


def test_8b_arch_whole_model_invariants(mods):
    """32 layers, Q4_K, fp16 KV: properties that hold by construction and need no CPU run."""
    ll, ops, syn = mods
    cfg = ll.MultiModelConfig(**dict(syn.LLAMA3_8B, max_seq=160))
    rt, _ = syn.build_runtime(cfg, orc.FMT_Q4_K, seed=4, kv_format=orc.FMT_F16)
    prompt = np.random.default_rng(12).integers(0, cfg.vocab, 20).astype(np.uint32)   # < 32 tokens: the token walk

    # graph replay = eager launches, token for token and bit for bit in the logits
    ll.set_graph_replay(rt, True)
    rt.reset(); rt.prefill(prompt)
    replay = ll.continue_greedy(rt, 24)
    logits_replay = rt.logits().copy()
    ll.set_graph_replay(rt, False)
    rt.reset(); rt.prefill(prompt)
    eager = ll.continue_greedy(rt, 24)
    assert replay == eager
    assert np.array_equal(logits_replay.view(np.uint32), rt.logits().view(np.uint32))
    ll.set_graph_replay(rt, True)

    # rollback into the prompt, walk its last token again and regenerate: the same stream (checkpoint = visible length)
    rt.set_visible(len(prompt) - 1)
    rt.advance(int(prompt[-1]))
    assert ll.continue_greedy(rt, 24) == replay

    # generate() = prefill + continue
    assert rt.generate(prompt, 24)[0] == replay

    # exact two-token decode with a one-layer draft commits the plain greedy stream
    dcfg = ll.MultiModelConfig(**dict(syn.LLAMA3_8B, n_layer=1, max_seq=160))
    draft, _ = syn.build_runtime(dcfg, orc.FMT_Q4_K, seed=5, kv_format=orc.FMT_F16)
    got, st = ll.generate_two_token(rt, draft, prompt, 24)
    assert got == replay
    assert st["passes"] <= st["committed_total"] <= 2 * st["passes"] and st["accepted_total"] == st["committed_total"] - st["passes"]
    # the target as its own draft: every proposal accepted
    twin, _ = syn.build_runtime(cfg, orc.FMT_Q4_K, seed=4, kv_format=orc.FMT_F16)
    got, st = ll.generate_two_token(rt, twin, prompt, 25)     # the prefill's token, then 12 passes of two
    assert got[:24] == replay and st["accepted_total"] == st["passes"] == 12
    twin.close(); draft.close()

    # a long prompt goes through the MFMA blocks; decoding on top of that cache stays a valid greedy stream of this
    # model: every next token is the argmax of the logits the runtime reports, and replays identically
    long_prompt = np.random.default_rng(13).integers(0, cfg.vocab, 100).astype(np.uint32)
    a = rt.generate(long_prompt, 16)[0]
    b = rt.generate(long_prompt, 16)[0]
    assert a == b
    rt.reset(); rt.prefill(long_prompt)
    for t in a[:6]:
        lg = rt.logits()
        assert int(np.argmax(lg)) == t == rt.select_greedy()      # first maximum = lowest index on ties
        rt.advance(t)
    rt.close()
