"""Greedy generation that ends at the stop token while its steps replay as one captured graph per token (the graph's own tail
kernel notices the token; the host looks once per 32 replays) against the host-driven loop: the same tokens - the stop token is
emitted and not consumed (RealModelInferenceEngine.swift:6385-6388) - and the same state afterwards, wherever the stop falls."""
import numpy as np
import pytest

import model_util as mu
from oracle import oracle as orc

pytestmark = pytest.mark.gpu

BASE = dict(n_layer=2, n_head=4, n_kv_head=2, d_model=256, head_dim=64, hidden_dim=512, vocab=512, max_seq=128)


@pytest.fixture(scope="module")
def llama():
    import espresso_amd.llama as ll
    import espresso_amd.ops as o
    o.init()
    return ll


def build(ll, packed, fmt, eos):
    rt = ll.LlamaRuntime(ll.MultiModelConfig(eos_token=eos, **BASE))
    ll.load_packed_weights(rt, packed, fmt)
    return rt


@pytest.mark.parametrize("fmt", [orc.FMT_Q8_0, orc.FMT_Q4_K])
def test_stop_token_inside_graph_replay(llama, fmt):
    ocfg = orc.LlamaConfig(gemv_inputs_fp16=True, **BASE)
    packed = mu.pack_weights(mu.random_weights(ocfg, 41, std=0.08), fmt)[0]
    prompt = [5, 6, 7, 8]
    free = build(llama, packed, fmt, -1)
    plain = free.generate(prompt, 100)[0]
    free.close()
    # stops at the first token, inside the first chunk of replays, at its edges (32, 33 tokens after the eager first step) and later
    for stop_at in (0, 1, 2, 17, 31, 32, 33, 34, 64, 65, 90):
        eos = plain[stop_at]
        first = plain.index(eos)
        results = []
        for graph in (True, False):
            rt = build(llama, packed, fmt, eos)
            llama.set_graph_replay(rt, graph)
            tokens, st = rt.generate(prompt, 100)
            state = (tokens, rt.visible(), rt.last_hidden().tobytes())
            # the runtime can go on from where the loop left it: consume the stop token and two more
            rt.advance(eos)
            more = [rt.select_greedy()]
            rt.advance(more[0]); more.append(rt.select_greedy())
            results.append(state + (more,))
            rt.close()
        assert results[0] == results[1], stop_at
        assert results[0][0] == plain[:first + 1]
        assert results[0][1] == len(prompt) + first           # the stop token was not consumed
    # a budget that ends before the stop token, and one that ends exactly on it
    eos = plain[40]
    first = plain.index(eos)
    for budget in (first, first + 1, first + 2):
        outs = []
        for graph in (True, False):
            rt = build(llama, packed, fmt, eos)
            llama.set_graph_replay(rt, graph)
            outs.append((rt.generate(prompt, budget)[0], rt.visible()))
            rt.close()
        assert outs[0] == outs[1] and outs[0][0] == plain[:min(budget, first + 1)]


def test_stop_token_on_a_reused_runtime_after_a_prompt_block(llama):
    """A runtime whose step graph already exists, given a prompt long enough for the block path (its row arrays then hold the
    block's rows, not the sequence's last row), with the stop token as the first, second or a later generated token: same tokens
    and same state (visible count, kept hidden row, logits, the tokens that follow) as the host-driven loop."""
    fmt = orc.FMT_Q8_0
    ocfg = orc.LlamaConfig(gemv_inputs_fp16=True, **BASE)
    packed = mu.pack_weights(mu.random_weights(ocfg, 43, std=0.08), fmt)[0]
    prompt = np.random.default_rng(3).integers(0, BASE["vocab"], 40).tolist()
    free = build(llama, packed, fmt, -1)
    plain = free.generate(prompt, 40)[0]
    free.close()
    for stop_at in (0, 1, 5):
        eos = plain[stop_at]
        first = plain.index(eos)
        results = []
        for graph in (True, False):
            rt = build(llama, packed, fmt, eos)
            llama.set_graph_replay(rt, graph)
            rt.generate([9, 10, 11, 12], 6)          # builds the step graphs; leaves another row in the row arrays
            rt.reset()
            tokens, _ = rt.generate(prompt, 40)
            state = (tokens, rt.visible(), rt.last_hidden().tobytes(), rt.logits().tobytes())
            rt.advance(eos)
            more = [rt.select_greedy()]
            rt.advance(more[0]); more.append(rt.select_greedy())
            results.append(state + (more,))
            rt.close()
        assert results[0] == results[1], stop_at
        assert results[0][0] == plain[:first + 1]
        assert results[0][1] == len(prompt) + first
