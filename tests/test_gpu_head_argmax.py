"""The output head whose epilogue is the arg-max (no logits stored): lowest index wins ties, as in the reference's
partitionedArgmax (RealModelInferenceEngine.swift:8219-8275) and its NEON argmax (neon_convert.c:36-101).

Ties are made exact by copying the packed bytes of the winning row of the head over other rows, in the same workgroup,
in neighbouring workgroups and far apart, at both benchmark vocabularies."""
import os

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
    return ll, ops, syn


def rebuilt(ll, cfg, packed, fmt, kv_format):
    rt = ll.LlamaRuntime(cfg, kv_format=kv_format)
    ll.load_packed_weights(rt, packed, fmt)
    return rt


@pytest.mark.parametrize("shape,fmt", [
    (dict(n_layer=1, n_head=12, n_kv_head=12, d_model=768, head_dim=64, hidden_dim=2048, vocab=32000, max_seq=64), orc.FMT_Q8_0),
    (dict(n_layer=1, n_head=12, n_kv_head=12, d_model=768, head_dim=64, hidden_dim=2048, vocab=32000, max_seq=64), orc.FMT_F16),
    (dict(n_layer=1, n_head=32, n_kv_head=8, d_model=4096, head_dim=128, hidden_dim=14336, vocab=128256, max_seq=64, rope_theta=500000.0), orc.FMT_Q4_K),
    (dict(n_layer=1, n_head=8, n_kv_head=8, d_model=512, head_dim=64, hidden_dim=512, vocab=1003, max_seq=64), orc.FMT_Q4_0),   # odd row count
])
def test_duplicated_rows_lowest_index_wins(mods, shape, fmt):
    ll, ops, syn = mods
    cfg = ll.MultiModelConfig(**shape)
    rt, packed = syn.build_runtime(cfg, fmt, seed=31, kv_format=orc.FMT_F16, keep_packed=True)
    prompt = [3, 1, 4, 1, 5]
    rt.prefill(prompt)
    logits = rt.logits()
    winner = int(np.argmax(logits))
    assert rt.select_greedy() == winner                      # fused head = first maximum of the stored logits
    rt.close()
    row_bytes = orc.format_bytes(fmt, cfg.d_model)
    head = np.array(packed["lm_head"], copy=True).reshape(cfg.vocab, row_bytes)
    v = cfg.vocab
    for case, dups in enumerate([
        [winner],                                             # no tie
        [min(winner + 1, v - 1), v - 1],                      # ties after the winner only
        [6, 7, 9, 16, 4001 % v, 17000 % v, v - 1],            # same row pair, same workgroup, next workgroup, far rows, last row
        [0, v // 2],
    ]):
        h = head.copy()
        h[dups] = head[winner]
        expect = min(dups + [winner])
        p2 = dict(packed, lm_head=h.reshape(-1))
        rt2 = rebuilt(ll, cfg, p2, fmt, orc.FMT_F16)
        rt2.prefill(prompt)
        lg = rt2.logits()
        assert np.all(lg[dups].view(np.uint32) == lg[winner].view(np.uint32))      # exact ties
        assert lg.max() == lg[winner]
        assert rt2.select_greedy() == expect, (case, dups, winner)
        # the captured step (head with arg-max epilogue -> tail kernel) commits the same token
        assert ll.continue_greedy(rt2, 2)[0] == expect
        # two rows at once (the verify step's head): both rows see the same tie
        rt2.reset(); rt2.prefill(prompt)
        got, _ = ll.generate_two_token(rt2, rebuilt(ll, cfg, p2, fmt, orc.FMT_F16), prompt, 3)
        assert got[0] == expect
        rt2.close()


def test_fused_head_switch_gives_the_same_tokens(mods):
    ll, ops, syn = mods
    cfg = ll.MultiModelConfig(n_layer=2, n_head=12, n_kv_head=12, d_model=768, head_dim=64, hidden_dim=2048, vocab=32000, max_seq=96)
    rt, packed = syn.build_runtime(cfg, orc.FMT_Q8_0, seed=5, keep_packed=True)
    prompt = list(range(10, 26))
    fused = rt.generate(prompt, 64)[0]
    rt.close()
    os.environ["ESPRESSO_HIP_FUSED_HEAD_ARGMAX"] = "0"
    try:
        plain = rebuilt(ll, cfg, packed, orc.FMT_Q8_0, orc.FMT_F32)
    finally:
        del os.environ["ESPRESSO_HIP_FUSED_HEAD_ARGMAX"]
    assert plain.generate(prompt, 64)[0] == fused
    plain.close()
