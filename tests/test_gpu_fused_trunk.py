"""The fused trunk kernel (one persistent launch per batch-1 step) against the separate kernels it fuses, on a
model of the Llama-3-8B layer shape with few layers.  The per-row-pair arithmetic is the same code in the same
order, so hidden states agree to the last bit; the separate kernels are the path the oracle tests pin."""
import numpy as np
import pytest

from oracle import oracle as orc

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def model():
    import espresso_amd.llama as ll
    import espresso_amd.ops as o
    import espresso_amd.synthetic as syn
    o.init()
    cfg = ll.MultiModelConfig(n_layer=3, n_head=32, n_kv_head=8, d_model=4096, head_dim=128, hidden_dim=14336, vocab=2048,
                              max_seq=320, norm_eps=1e-5, rope_theta=500000.0)
    rt, _ = syn.build_runtime(cfg, orc.FMT_Q4_K, seed=11, std=0.02, kv_format=orc.FMT_F16)
    # the trunk kernel's attention phase splits the prefix and merges in its own pass: compare it with the
    # separate kernels in that same form, not with the one-launch attention merged by the wo GEMV
    assert not ll.set_merged_attention(rt, False)
    return ll, rt


def _run(ll, rt, fused, prompt, steps):
    ll.set_fused_trunk(rt, fused)
    ll.set_graph_replay(rt, False)
    rt.reset()
    rt.prefill(prompt)
    hidden = [rt.last_hidden().copy()]
    tokens = []
    for _ in range(steps):
        t = rt.select_greedy()
        tokens.append(t)
        rt.advance(t)
        hidden.append(rt.last_hidden().copy())
    return tokens, hidden


def test_fused_trunk_is_used_and_matches_separate_kernels(model):
    ll, rt = model
    assert ll.fused_trunk_status(rt) == (False, 0)       # opt-in: measured slower than the separate kernels
    ll.set_fused_trunk(rt, True)
    assert ll.fused_trunk_status(rt) == (True, 0)
    prompt = np.random.default_rng(1).integers(0, 2048, 20).tolist()    # per-token prefill: every prompt token runs the trunk
    tok_f, hid_f = _run(ll, rt, True, prompt, 12)
    assert ll.fused_trunk_status(rt) == (True, 0)
    tok_s, hid_s = _run(ll, rt, False, prompt, 12)
    assert tok_f == tok_s
    for a, b in zip(hid_f, hid_s):
        assert np.isfinite(a).all()
        assert np.array_equal(a.view(np.uint32), b.view(np.uint32)), np.abs(a - b).max()


def test_fused_trunk_long_context_and_graph_replay(model):
    ll, rt = model
    prompt = np.random.default_rng(2).integers(0, 2048, 280).tolist()   # block prefill, then decode at context 280+
    ll.set_fused_trunk(rt, True)
    ll.set_graph_replay(rt, True)
    rt.reset()
    rt.prefill(prompt)
    got = ll.continue_greedy(rt, 24)
    h_fused = rt.last_hidden().copy()
    assert ll.fused_trunk_status(rt) == (True, 0)
    ll.set_fused_trunk(rt, False)
    ll.set_graph_replay(rt, False)
    rt.reset()
    rt.prefill(prompt)
    want = ll.continue_greedy(rt, 24)
    assert got == want
    assert np.array_equal(h_fused.view(np.uint32), rt.last_hidden().view(np.uint32))
    ll.set_graph_replay(rt, True)
