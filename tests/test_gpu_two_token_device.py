"""The exact two-token loop with its passes on the device (one captured graph per pass, no host decision in between)
against the same loop driven from the host (graph replay switched off on the target): the same tokens, the same six
counters of the reference loop (RealModelInferenceEngine.swift:6109-6186) and the same state left in both models,
for drafts that never, sometimes and always agree, with stop tokens, odd and even budgets and the end of the context."""
import numpy as np
import pytest

import model_util as mu
from oracle import oracle as orc

pytestmark = pytest.mark.gpu

BASE = dict(n_head=4, n_kv_head=2, d_model=256, head_dim=64, hidden_dim=512, vocab=512)
COUNTERS = ("passes", "committed_total", "accepted_total", "reference_passes", "reference_committed_total", "reference_accepted_total")


@pytest.fixture(scope="module")
def llama():
    import espresso_amd.llama as ll
    import espresso_amd.ops as o
    o.init()
    return ll


def build(ll, packed, fmt, n_layer, max_seq, eos=-1):
    cfg = ll.MultiModelConfig(n_layer=n_layer, max_seq=max_seq, eos_token=eos, **BASE)
    rt = ll.LlamaRuntime(cfg)
    ll.load_packed_weights(rt, dict(packed, layers=packed["layers"][:n_layer]), fmt)
    return rt


def weights(fmt, seed, n_layer, upper_scale=1.0):
    """Random model whose layers above the first are scaled by `upper_scale` in their output projections: 0 makes the first layer
    alone an exact draft of the whole model, small values a draft that agrees most of the time."""
    ocfg = orc.LlamaConfig(gemv_inputs_fp16=True, n_layer=n_layer, max_seq=64, **BASE)
    w = mu.random_weights(ocfg, seed, std=0.08)
    for L in w["layers"][1:]:
        L["wo"] *= upper_scale
        L["w2"] *= upper_scale
    return mu.pack_weights(w, fmt)[0]


def both_ways(ll, target, draft, prompt, budget, reference_accounting=True):
    results = []
    for on_device in (True, False):
        ll.set_graph_replay(target, on_device)
        target.reset(); draft.reset()
        tokens, st = ll.generate_two_token(target, draft, prompt, budget, reference_accounting)
        results.append((tokens, {k: st[k] for k in COUNTERS}, target.visible(), draft.visible(), target.last_hidden(), draft.last_hidden(),
                        target.select_greedy(), draft.select_greedy()))
    ll.set_graph_replay(target, True)
    dev, host = results
    assert dev[0] == host[0]
    assert dev[1] == host[1], (dev[1], host[1])
    assert dev[2:4] == host[2:4]                                     # visible token counts of target and draft
    assert np.array_equal(dev[4], host[4]) and np.array_equal(dev[5], host[5])   # kept hidden states, bit for bit
    assert dev[6:] == host[6:]
    return dev[0], dev[1]


@pytest.mark.parametrize("fmt", [orc.FMT_Q8_0, orc.FMT_Q4_K])
def test_device_passes_equal_the_host_loop(llama, fmt):
    prompt = [7, 8, 9, 10, 11]
    seen = set()
    for label, upper in (("never agrees", None), ("sometimes", 0.15), ("always", 0.0)):
        if upper is None:
            target = build(llama, weights(fmt, 21, 3), fmt, 3, 64)
            draft = build(llama, weights(fmt, 22, 1), fmt, 1, 64)
        else:
            packed = weights(fmt, 23, 3, upper)
            target, draft = build(llama, packed, fmt, 3, 64), build(llama, packed, fmt, 1, 64)
        plain = target.generate(prompt, 50)[0]
        for budget in (1, 2, 3, 4, 5, 8, 21, 50):
            for ref in (True, False):
                tokens, st = both_ways(llama, target, draft, prompt, budget, ref)
                assert tokens == plain[:budget], (label, budget)
                if budget == 50 and ref:
                    rate = st["accepted_total"] / st["passes"]
                    seen.add(label)
                    if label == "never agrees": assert rate < 0.2
                    if label == "always":      # 49 tokens after the first: 24 accepted passes and a last pass with one token of budget
                        assert (st["passes"], st["accepted_total"], st["committed_total"]) == (25, 24, 49)
                    if label == "sometimes": assert 0.1 < rate < 1.0, rate
        target.close(); draft.close()
    assert seen == {"never agrees", "sometimes", "always"}


def test_stop_token_and_context_end_on_the_device(llama):
    fmt = orc.FMT_Q8_0
    packed = weights(fmt, 23, 3, 0.15)
    prompt = [7, 8, 9, 10, 11]
    probe = build(llama, packed, fmt, 3, 64)
    plain = probe.generate(prompt, 40)[0]
    probe.close()
    # every position of the stream once as the stop token: the stop may fall on the first or the second token of a pass
    for stop_at in range(0, 12):
        eos = plain[stop_at]
        first = plain.index(eos)
        target, draft = build(llama, packed, fmt, 3, 64, eos=eos), build(llama, packed, fmt, 1, 64, eos=eos)
        tokens, _ = both_ways(llama, target, draft, prompt, 40)
        assert tokens == plain[:first + 1]
        target.close(); draft.close()
    # the context ends before the budget does (prompt 5 + generated tokens fill max_seq)
    for max_seq in (12, 13, 20):
        target, draft = build(llama, packed, fmt, 3, max_seq), build(llama, packed, fmt, 1, max_seq)
        tokens, _ = both_ways(llama, target, draft, prompt, 40)
        assert tokens == plain[:max_seq - len(prompt)]
        target.close(); draft.close()
    # a draft with a shorter context than the target bounds the loop as well (:6040-6047)
    target, draft = build(llama, packed, fmt, 3, 64), build(llama, packed, fmt, 1, 17)
    tokens, _ = both_ways(llama, target, draft, prompt, 40)
    assert tokens == plain[:17 - len(prompt)]
    target.close(); draft.close()


def build_batch(ll, packed, fmt, n_layer, max_seq, n_seq):
    cfg = ll.MultiModelConfig(n_layer=n_layer, max_seq=max_seq, **BASE)
    rt = ll.LlamaRuntime(cfg, max_sequences=n_seq)
    ll.load_packed_weights(rt, dict(packed, layers=packed["layers"][:n_layer]), fmt)
    return rt


@pytest.mark.parametrize("n_seq", [1, 3, 16])
def test_lock_step_loops_on_the_device_equal_the_host_loops(llama, n_seq):
    """generate_batch (plain greedy and the exact two-token loop over several sequences): passes replayed as graphs with the
    per-sequence variables on the device against the host-driven loops - the same streams, counters and visible counts."""
    fmt = orc.FMT_Q8_0
    rng = np.random.default_rng(n_seq)
    prompts = [rng.integers(0, BASE["vocab"], int(rng.integers(3, 9))).astype(np.uint32) for _ in range(n_seq)]
    for label, upper in (("never agrees", None), ("sometimes", 0.15), ("always", 0.0)):
        if upper is None:
            target = build_batch(llama, weights(fmt, 21, 3), fmt, 3, 64, n_seq)
            draft = build_batch(llama, weights(fmt, 22, 1), fmt, 1, 64, n_seq)
        else:
            packed = weights(fmt, 23, 3, upper)
            target, draft = build_batch(llama, packed, fmt, 3, 64, n_seq), build_batch(llama, packed, fmt, 1, 64, n_seq)
        for budget in (1, 2, 3, 4, 9, 30):
            runs = {}
            for on_device in (True, False):
                for d in (None, draft):
                    llama.set_graph_replay(target, on_device)
                    target.reset(); draft.reset()
                    toks, st = llama.generate_batch(target, prompts, budget, draft=d)
                    runs[(on_device, d is not None)] = (toks, (st["passes"], st["committed_total"], st["accepted_total"]),
                                                        [target.visible(s) for s in range(n_seq)], [draft.visible(s) for s in range(n_seq)])
            llama.set_graph_replay(target, True)
            assert runs[(True, False)] == runs[(False, False)], (label, budget, "plain greedy")
            assert runs[(True, True)] == runs[(False, True)], (label, budget, "two-token")
            assert runs[(True, True)][0] == runs[(True, False)][0]                  # the exact loop gives the greedy streams
            assert all(len(t) == budget for t in runs[(True, True)][0])
            if label == "always" and budget == 30:
                passes, committed, accepted = runs[(True, True)][1]
                assert accepted == 14 * n_seq and committed == 29 * n_seq and passes == 15
        target.close(); draft.close()


def test_device_loop_session_is_reused_and_rebuilt(llama):
    """The target keeps the loop's device state, log and captured passes between calls: the same pair again (other budgets, long
    enough for the four-pass graph and too short for it), another draft, the first draft again, and a pair whose kernels changed
    (merged attention switched off and on) all give the host-driven loop's result."""
    fmt = orc.FMT_F16
    packed = weights(fmt, 31, 3, upper_scale=0.05)
    other = weights(fmt, 32, 3, upper_scale=1.0)
    target = build(llama, packed, fmt, 3, 64)
    draft_a, draft_b = build(llama, packed, fmt, 1, 64), build(llama, other, fmt, 1, 64)
    prompt = [7, 8, 9, 10, 11]
    seen = []
    for draft, budget in ((draft_a, 40), (draft_a, 9), (draft_a, 33), (draft_b, 40), (draft_a, 40), (draft_b, 5)):
        tokens, _ = both_ways(llama, target, draft, prompt, budget)
        seen.append(tokens)
    assert seen[0] == seen[4] and seen[0][:9] == seen[1] and seen[3][:5] == seen[5] and seen[0] == seen[3]   # exact: the draft does not matter
    for enabled in (False, True):
        llama.set_merged_attention(draft_a, enabled)
        llama.set_merged_attention(target, enabled)
        tokens, _ = both_ways(llama, target, draft_a, prompt, 40)
        assert tokens == seen[0]
    for rt in (target, draft_a, draft_b):
        rt.close()
