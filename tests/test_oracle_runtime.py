"""Pins the oracle's stateful runtime and its two generation loops (no GPU)."""
import numpy as np
import pytest

import model_util as mu
import numpy_ref as ref
from oracle import oracle as orc


def tiny_cfg(**kw):
    base = dict(n_layer=2, n_head=4, n_kv_head=2, d_model=32, head_dim=8, hidden_dim=48, vocab=64, max_seq=24,
                norm_eps=1e-5, rope_theta=10000.0)
    base.update(kw)
    return orc.LlamaConfig(**base)


def test_forward_matches_float64_decoder_gqa():
    cfg = tiny_cfg()
    w = mu.random_weights(cfg, seed=11, std=0.3, norm_jitter=0.1)
    rt = mu.load_oracle(cfg, w)
    f64 = ref.Llama64(cfg, w)
    toks = [3, 17, 60, 5, 5, 41, 0, 63, 22]
    assert rt.prefill(toks[:1]) == 0
    h = f64.forward(toks[0])
    for t in toks[1:]:
        assert np.allclose(rt.last_hidden(), h, rtol=2e-4, atol=2e-5)
        assert np.allclose(rt.logits(), f64.logits(h), rtol=2e-4, atol=2e-4)
        assert rt.select_greedy() == int(np.argmax(rt.logits()))
        assert rt.advance(t) == 0
        h = f64.forward(t)
    assert rt.visible == len(toks)


def test_tiny_llama_constant_weights_fixture():
    """The reference's tiny-llama test model (RealModelInferenceTests.swift:3199-3245):
    1 layer, 2 heads / 1 kv head, d=8, headDim 4, hidden 16, vocab 32, constant weights."""
    cfg = orc.LlamaConfig(n_layer=1, n_head=2, n_kv_head=1, d_model=8, head_dim=4, hidden_dim=16, vocab=32,
                          max_seq=16, norm_eps=1e-6)
    sh = mu.matrix_shapes(cfg)
    const = {"wq": 0.03125, "wk": 0.015625, "wv": 0.0234375, "wo": 0.02734375, "w1": 0.01953125,
             "w2": 0.01171875, "w3": 0.017578125}
    rng = np.random.default_rng(0)
    w = {"embedding": rng.normal(0, 1, (32, 8)).astype(np.float32), "final_norm": np.ones(8, np.float32),
         "lm_head": rng.normal(0, 1, (32, 8)).astype(np.float32),
         "layers": [dict({k: np.full(sh[k], v, np.float32) for k, v in const.items()},
                         rms_att=np.ones(8, np.float32), rms_ffn=np.ones(8, np.float32))]}
    rt = mu.load_oracle(cfg, w)
    f64 = ref.Llama64(cfg, w)
    for i, t in enumerate([1, 9, 30, 4]):
        assert rt.advance(t) == 0
        h = f64.forward(t)
        assert np.allclose(rt.last_hidden(), h, rtol=1e-5, atol=1e-6)
        # closed form: constant matrices make every projection a multiple of sum(normed)
        if i == 0:
            x = w["embedding"][t].astype(np.float64)
            n = x / np.sqrt((x * x).mean() + 1e-6)
            v = 0.0234375 * n.sum()                       # every v channel; one token => ctx = v
            p = x + 0.02734375 * 8 * v
            f = p / np.sqrt((p * p).mean() + 1e-6)
            g, u = 0.01953125 * f.sum(), 0.017578125 * f.sum()
            want = p + 0.01171875 * 16 * (g / (1 + np.exp(-g)) * u)
            assert np.allclose(rt.last_hidden(), want, rtol=1e-5, atol=1e-6)


def test_errors_and_limits():
    cfg = tiny_cfg(max_seq=4)
    rt = mu.load_oracle(cfg, mu.random_weights(cfg, 1))
    assert rt.prefill([]) == -1                               # empty prompt (:638-640)
    assert rt.prefill([1, 2, 3, 4]) == 0
    assert rt.advance(1) == -2                                # position beyond context (:673-677)
    rt.reset()
    assert rt.advance(cfg.vocab) == -3                        # token outside vocab (:687-689)
    with pytest.raises(ValueError):
        orc.LlamaRuntime(tiny_cfg(n_head=3, n_kv_head=2))     # nHead % nKVHead (:7615-7634)


def test_checkpoint_rollback_restores_state():
    cfg = tiny_cfg()
    rt = mu.load_oracle(cfg, mu.random_weights(cfg, 2, std=0.3))
    rt.prefill([1, 2, 3])
    ck = rt.capture()
    before = rt.last_hidden()
    rt.advance(9); rt.advance(10)
    rt.rollback(ck)
    orc.LlamaRuntime.free_checkpoint(ck)
    assert rt.visible == 3 and np.array_equal(rt.last_hidden(), before)
    rt.advance(7)
    a = rt.last_hidden()
    rt2 = mu.load_oracle(cfg, mu.random_weights(cfg, 2, std=0.3))
    rt2.prefill([1, 2, 3, 7])
    assert np.array_equal(a, rt2.last_hidden())
    # rollback by lowering the visible length alone gives the same continuation
    rt2.advance(30); rt2.set_visible(3); rt2.advance(7)
    assert np.array_equal(a, rt2.last_hidden())


def test_rounding_switches():
    cfg = tiny_cfg()
    w = mu.random_weights(cfg, 4, std=0.3)
    base = mu.load_oracle(cfg, w); base.prefill([5, 6, 7])
    for flag in ("round_intermediates_fp16", "gemv_inputs_fp16", "kv_fp16"):
        rt = mu.load_oracle(tiny_cfg(**{flag: True}), w); rt.prefill([5, 6, 7])
        diff = np.abs(rt.last_hidden() - base.last_hidden()).max()
        assert 0 < diff < 2e-2, flag
    rt = mu.load_oracle(tiny_cfg(round_intermediates_fp16=True), w); rt.prefill([5, 6, 7])
    h = rt.last_hidden()
    assert np.array_equal(h, h.astype(np.float16).astype(np.float32))


def test_generate_stops_and_matches_stepwise():
    cfg = tiny_cfg(max_seq=12)
    w = mu.random_weights(cfg, 6, std=0.3)
    rt = mu.load_oracle(cfg, w)
    prompt = [1, 2, 3, 4]
    toks = rt.generate(prompt, 100)
    assert len(toks) == 8                                      # min(maxTokens, maxSeq - promptLen)
    step = mu.load_oracle(cfg, w); step.prefill(prompt)
    want = []
    for _ in range(8):
        t = step.select_greedy(); want.append(t)
        if len(want) < 8:
            step.advance(t)
    assert toks == want
    assert rt.generate(prompt, 3) == want[:3]
    # EOS is appended, then generation stops (:6385-6388)
    eos_cfg = tiny_cfg(max_seq=12, eos_token=want[2])
    assert mu.load_oracle(eos_cfg, w).generate(prompt, 100) == want[:3]
    toks2, margin = mu.load_oracle(cfg, w).generate(prompt, 8, with_margin=True)
    assert toks2 == want and margin > 0


def bigram_model(d_model=128, vocab=128, layers=1):
    """LocalBigramArtifactBuilder (Sources/Espresso/LocalBigramArtifactBuilder.swift:46-205):
    one-hot embeddings, classifier[next, cur] = 10, zero trunk."""
    corpus = [35, 105, 110, 116, 32, 105, 110, 116, 32]
    cfg = orc.LlamaConfig(n_layer=layers, n_head=2, n_kv_head=2, d_model=d_model, head_dim=d_model // 2,
                          hidden_dim=16, vocab=vocab, max_seq=32)
    sh = mu.matrix_shapes(cfg)
    emb = np.zeros((vocab, d_model), np.float32)
    emb[np.arange(min(vocab, d_model)), np.arange(min(vocab, d_model))] = 1
    head = np.zeros((vocab, d_model), np.float32)
    counts = {}
    for a, b in zip(corpus[:-1], corpus[1:]):
        counts.setdefault(a, {}).setdefault(b, 0)
        counts[a][b] += 1
    for cur, nxt in counts.items():
        best = max(nxt.items(), key=lambda kv: (kv[1], -kv[0]))[0]
        head[best, cur] = 10
    w = {"embedding": emb, "final_norm": np.ones(d_model, np.float32), "lm_head": head,
         "layers": [dict({k: np.zeros(sh[k], np.float32) for k in mu.MATRICES},
                         rms_att=np.ones(d_model, np.float32), rms_ffn=np.ones(d_model, np.float32))
                    for _ in range(layers)]}
    return cfg, w


def test_local_bigram_golden_tokens():
    """Golden: [35] -> [105, 110, 116, 32] (GenerationHarnessTests.swift:781-849)."""
    cfg, w = bigram_model()
    assert mu.load_oracle(cfg, w).generate([35], 4) == [105, 110, 116, 32]
    toks, st = orc.generate_two_token(mu.load_oracle(cfg, w), mu.load_oracle(cfg, w), [35], 4)
    assert toks == [105, 110, 116, 32]
    # CPU loop accounting (:6109-6163): first token outside the passes; pass 1 commits 2 and
    # accepts both proposals; pass 2 has budget 1: commits 1, accepts 1.
    assert st == {"passes": 2, "committed_total": 3, "accepted_total": 3}


def test_two_token_stream_equals_plain_greedy():
    full_cfg = tiny_cfg(n_layer=3, max_seq=40)
    draft_cfg = tiny_cfg(n_layer=1, max_seq=40)
    wf, wd = mu.random_weights(full_cfg, 21, std=0.3), mu.random_weights(draft_cfg, 22, std=0.3)
    prompt = [7, 8, 9, 10, 11]
    for budget in (1, 2, 3, 10, 35, 100):
        plain = mu.load_oracle(full_cfg, wf).generate(prompt, budget)
        toks, st = orc.generate_two_token(mu.load_oracle(full_cfg, wf), mu.load_oracle(draft_cfg, wd), prompt, budget)
        assert toks == plain
        assert st["committed_total"] == max(len(toks) - 1, 0)
        assert 0 <= st["accepted_total"] <= st["committed_total"]
    # a draft identical to the target accepts every proposal
    toks, st = orc.generate_two_token(mu.load_oracle(full_cfg, wf), mu.load_oracle(full_cfg, wf), prompt, 21)
    assert st["accepted_total"] == st["committed_total"] == 20 and st["passes"] == 10
