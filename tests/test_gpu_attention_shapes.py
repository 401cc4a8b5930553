"""The single-query attention kernel picks wavefronts x chunks per workgroup from the context size (launch_attention_partials).
Every shape of the table runs here against the oracle, with prefixes that need one and several passes of a wavefront's loop and
with positions on both sides of the pass boundaries; fp16 and fp32 KV caches."""
import numpy as np
import pytest

from oracle import oracle as orc
from test_gpu_full_size import oracle_from_packed

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def mods():
    import espresso_amd.llama as ll
    import espresso_amd.ops as ops
    import espresso_amd.synthetic as syn
    ops.init()
    return ll, ops, syn


# (head size, context size) -> (wavefronts, chunks): 64: <=256 (2,2), <=512 (2,4), <=1024 (4,4), above (8,4); 128: <=256 (2,4), <=512 (4,4), above (8,6)
@pytest.mark.parametrize("head_dim,max_seq,prompt_len,kv_fp16", [
    (64, 256, 140, False), (64, 512, 300, True), (64, 1024, 700, False), (64, 1536, 1200, True),
    (128, 256, 200, True), (128, 512, 400, False), (128, 1024, 900, True),
])
def test_attention_shape_for_the_context_size_matches_oracle(mods, head_dim, max_seq, prompt_len, kv_fp16):
    ll, ops, syn = mods
    n_head, n_kv = 4, 2
    cfg = ll.MultiModelConfig(n_layer=2, n_head=n_head, n_kv_head=n_kv, d_model=n_head * head_dim, head_dim=head_dim, hidden_dim=512,
                              vocab=512, max_seq=max_seq, norm_eps=1e-5, rope_theta=10000.0, name="attention-shapes")
    g, packed = syn.build_runtime(cfg, orc.FMT_F16, seed=head_dim + max_seq, std=0.05, keep_packed=True,
                                  kv_format=orc.FMT_F16 if kv_fp16 else orc.FMT_F32)
    assert ll.set_merged_attention(g, True)       # the kernel under test is the one the decode step uses
    o = oracle_from_packed(cfg, packed, orc.FMT_F16, 2, kv_fp16, max_seq)
    prompt = [int(t) for t in np.random.default_rng(prompt_len).integers(0, cfg.vocab, prompt_len)]
    o.prefill(prompt)
    ll.set_matrix_prefill(g, False)          # every position through the single-query kernel, like the oracle's walk
    g.prefill(np.asarray(prompt, np.uint32))
    worst = 0.0
    for step in range(12):
        ho, hg = o.last_hidden(), g.last_hidden()
        assert np.abs(ho - hg).max() <= 2e-3 * max(1.0, np.abs(ho).max()), (step, np.abs(ho - hg).max())
        worst = max(worst, float(np.abs(o.logits() - g.logits()).max()))
        assert worst <= 2e-2
        t = o.select_greedy()
        o.advance(t)
        g.advance(t)
    g.close()
