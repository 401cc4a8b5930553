"""GPU: the engine built from a weight directory (BLOBFILEs, float32 sidecars, packed sidecars), the
GGUF front door, the draft selection through the environment, and the exact two-token harness."""
import json
import os

import numpy as np
import pytest

import model_util as mu
from gguf_writer import gguf_model, write_gguf
from oracle import oracle as orc

pytestmark = pytest.mark.gpu

KW = dict(n_layer=2, n_head=4, n_kv_head=2, d_model=256, head_dim=64, hidden_dim=512, vocab=512, max_seq=48)
PROMPT = [3, 141, 59, 26, 5]


@pytest.fixture(scope="module")
def E():
    import espresso_amd.engine as eng
    import espresso_amd.ops as ops
    ops.init()
    return eng


def gpu_cfg(kw, **extra):
    import espresso_amd.llama as ll
    return ll.MultiModelConfig(**kw, **extra)


def write_weight_dir(root, kw, w, f32_sidecars=False, packed_fmt=None, names=("embedding", "final_norm", "lm_head")):
    """Writes the reference's directory layout; returns the fp32 values an exact CPU run would see."""
    import espresso_amd.engine as eng
    os.makedirs(os.path.join(root, "embeddings"), exist_ok=True)
    seen = {"layers": []}

    def put(rel, a, matrix):
        path = os.path.join(root, rel)
        open(path, "wb").write(orc.blob_build(a))
        val = a.astype(np.float16).astype(np.float32)
        if f32_sidecars:
            a.astype("<f4").tofile(path[:-4] + ".float32.bin")
            val = a
        if matrix and packed_fmt is not None:
            blocks = orc.quantize(packed_fmt, a)
            tag = {orc.FMT_Q8_0: "q8_0", orc.FMT_Q4_0: "q4_0", orc.FMT_Q4_K: "q4_k"}[packed_fmt]
            blocks.tofile(path[:-4] + f".{tag}.bin")
            val = orc.dequantize(packed_fmt, blocks, a.size).reshape(a.shape)
        return val

    seen["embedding"] = put("embeddings/token.bin", w["embedding"], False)
    seen["final_norm"] = put("rms_final.bin", w["final_norm"], False)
    seen["lm_head"] = put("lm_head.bin", w["lm_head"], True)
    for l, L in enumerate(w["layers"]):
        os.makedirs(os.path.join(root, "layers", str(l)), exist_ok=True)
        seen["layers"].append({k: put(f"layers/{l}/{k}.bin", a, k in mu.MATRICES) for k, a in L.items()})
    eng.write_metadata(gpu_cfg(kw), os.path.join(root, "metadata.json"))
    return seen


def oracle_tokens(kw, seen, prompt, n, **flags):
    return mu.load_oracle(orc.LlamaConfig(gemv_inputs_fp16=True, **kw, **flags), seen).generate(prompt, n)


@pytest.mark.parametrize("mode", ["blobs", "float32_sidecars", "packed_q8_0", "packed_q4_k"])
def test_engine_from_weight_directory(E, tmp_path, mode):
    w = mu.random_weights(orc.LlamaConfig(**KW), 41, std=0.08, norm_jitter=0.05)
    seen = write_weight_dir(str(tmp_path), KW, w, f32_sidecars=mode == "float32_sidecars",
                            packed_fmt={"packed_q8_0": orc.FMT_Q8_0, "packed_q4_k": orc.FMT_Q4_K}.get(mode))
    e = E.RealModelInferenceEngine(gpu_cfg(KW), str(tmp_path), tokenizer_dir=None)
    toks, res = e.generate(PROMPT, 20)
    assert toks == oracle_tokens(KW, seen, PROMPT, 20)
    assert res["token_count"] == 20 and res["exact_head_backend"] == "hip_gemv_argmax" and res["has_two_token_stats"] == 0
    assert res["compile_time_ms"] > 0 and res["tokens_per_second"] > 0
    # maxTokens is clipped to the context (RealModelInferenceEngine.swift:1425-1426); zero budget returns nothing
    assert len(e.generate(PROMPT, 1000)[0]) == KW["max_seq"] - len(PROMPT)
    assert e.generate(PROMPT, 0)[0] == []
    e.close()


def test_engine_errors(E, tmp_path):
    import espresso_amd._lib as lib
    w = mu.random_weights(orc.LlamaConfig(**KW), 42, std=0.08)
    write_weight_dir(str(tmp_path), KW, w)
    with pytest.raises(lib.EspressoError, match="missing path"):
        E.RealModelInferenceEngine(gpu_cfg(KW), str(tmp_path / "nope"))
    with pytest.raises(lib.EspressoError, match="does not match config"):
        E.RealModelInferenceEngine(gpu_cfg(dict(KW, n_layer=3)), str(tmp_path))                 # metadata.json disagrees
    e = E.RealModelInferenceEngine(gpu_cfg(KW), str(tmp_path))
    with pytest.raises(lib.EspressoError, match="must not be empty"):
        e.generate([], 4)
    with pytest.raises(lib.EspressoError, match="maxTokens"):
        e.generate(PROMPT, -1)
    with pytest.raises(lib.EspressoError, match="temperature"):
        e.generate(PROMPT, 4, temperature=float("nan"))
    with pytest.raises(lib.EspressoError, match="does not fit context"):
        e.generate(list(range(KW["max_seq"])), 4)
    e.close()
    os.remove(tmp_path / "layers" / "1" / "w2.bin")
    with pytest.raises(lib.EspressoError, match="missing weight file"):
        E.RealModelInferenceEngine(gpu_cfg(KW), str(tmp_path))
    os.remove(tmp_path / "lm_head.bin")
    with pytest.raises(lib.EspressoError, match="missing lm head"):
        E.RealModelInferenceEngine(gpu_cfg(KW), str(tmp_path))


def test_exact_two_token_draft_through_environment(E, tmp_path):
    """ESPRESSO_BUNDLE_DRAFT_* -> descriptor JSON -> draft directory (RealModelInferenceEngine.swift:5324-5390)."""
    import espresso_amd._lib as lib
    root = tmp_path / "bundle"
    wdir = root / "weights"
    full_kw, draft_kw = dict(KW, n_layer=3), dict(KW, n_layer=1)
    wf = mu.random_weights(orc.LlamaConfig(**full_kw), 51, std=0.08)
    wd = mu.random_weights(orc.LlamaConfig(**draft_kw), 52, std=0.08)
    os.makedirs(wdir)
    seen_f = write_weight_dir(str(wdir), full_kw, wf)
    seen_d = write_weight_dir(str(wdir / "draft"), draft_kw, wd)
    (root / "draft.json").write_text(json.dumps({"model_dir": "draft", "tokenizer_dir": None, "model_id": "d"}))
    env = {"ESPRESSO_BUNDLE_DRAFT_KIND": "exact_two_token", "ESPRESSO_BUNDLE_DRAFT_HORIZON": "2",
           "ESPRESSO_BUNDLE_DRAFT_ARTIFACT_REF": "draft.json"}
    e = E.RealModelInferenceEngine(gpu_cfg(full_kw), str(wdir))
    plain, _ = e.generate(PROMPT, 24)
    toks, res = e.generate(PROMPT, 24, environment=env)
    of = mu.load_oracle(orc.LlamaConfig(gemv_inputs_fp16=True, **full_kw), seen_f)
    od = mu.load_oracle(orc.LlamaConfig(gemv_inputs_fp16=True, **draft_kw), seen_d)
    want, st = orc.generate_two_token(of, od, PROMPT, 24)
    assert toks == plain == want
    assert res["exact_head_backend"] == "hip_exact_two_token_draft" and res["has_two_token_stats"] == 1
    assert res["committed_exact_tokens_per_pass"] == pytest.approx(st["committed_total"] / st["passes"])
    assert res["accepted_future_tokens_per_pass"] == pytest.approx(st["accepted_total"] / st["passes"])
    for bad_env, message in [(dict(env, ESPRESSO_BUNDLE_DRAFT_HORIZON="3"), "horizon == 2"),
                             (dict(env, ESPRESSO_BUNDLE_DRAFT_ARTIFACT_REF="../x.json"), "escapes bundle root"),
                             (dict(env, ESPRESSO_BUNDLE_DRAFT_ARTIFACT_REF="none.json"), "is missing"),
                             ({"ESPRESSO_BUNDLE_DRAFT_KIND": "exact_two_token"}, "requires ESPRESSO_BUNDLE_DRAFT_ARTIFACT_REF")]:
        with pytest.raises(lib.EspressoError, match=message):
            e.generate(PROMPT, 4, environment=bad_env)
    (root / "draft.json").write_text(json.dumps({"model_dir": "../elsewhere"}))
    with pytest.raises(lib.EspressoError, match="escapes weights root"):
        e.generate(PROMPT, 4, environment=env)
    small = dict(draft_kw, vocab=256)
    write_weight_dir(str(wdir / "other"), small, mu.random_weights(orc.LlamaConfig(**small), 53, std=0.08))
    (root / "draft.json").write_text(json.dumps({"model_dir": "other"}))
    with pytest.raises(lib.EspressoError, match="vocab mismatch"):
        e.generate(PROMPT, 4, environment=env)
    e.close()


@pytest.mark.parametrize("arch,fmt,tied", [("llama", orc.FMT_Q8_0, False), ("llama", orc.FMT_Q4_K, True), ("qwen2", orc.FMT_Q4_0, False)])
def test_gguf_prepare_then_engine(E, tmp_path, arch, fmt, tied):
    w = mu.random_weights(orc.LlamaConfig(**KW), 61, std=0.08, norm_jitter=0.05)
    path = str(tmp_path / "m.gguf")
    seen = gguf_model(path, KW, w, arch, fmt, tied=tied, interleave_qk=arch == "llama")
    cfg, wdir, count = E.gguf_prepare(path, str(tmp_path / "prepared"))
    assert count == 2 + (0 if tied else 1) + 9 * KW["n_layer"]
    assert (cfg.n_layer, cfg.n_head, cfg.n_kv_head, cfg.d_model, cfg.head_dim, cfg.hidden_dim, cfg.vocab, cfg.max_seq, cfg.eos_token) == \
           (2, 4, 2, 256, 64, 512, 512, 48, 2)
    assert cfg.name == arch and cfg.rope_theta == 10000.0
    assert json.load(open(os.path.join(wdir, "metadata.json")))["vocab"] == 512
    tag = {orc.FMT_Q8_0: "q8_0", orc.FMT_Q4_0: "q4_0", orc.FMT_Q4_K: "q4_k"}[fmt]
    assert os.path.exists(os.path.join(wdir, f"layers/0/wq.{tag}.bin")) and not os.path.exists(os.path.join(wdir, "layers/0/wq.bin"))
    assert os.path.exists(os.path.join(wdir, "rms_final.float32.bin"))
    assert os.path.exists(os.path.join(wdir, "lm_head.bin" if tied else f"lm_head.{tag}.bin"))
    e = E.RealModelInferenceEngine(cfg, wdir)
    cfg.eos_token = -1
    toks, _ = e.generate(PROMPT, 16)
    okw = dict(KW, eos_token=2)
    assert toks == oracle_tokens(okw, seen, PROMPT, 16)
    e.close()


def test_gguf_prepare_can_emit_reference_blobfiles(E, tmp_path):
    w = mu.random_weights(orc.LlamaConfig(**KW), 62, std=0.08)
    path = str(tmp_path / "m.gguf")
    seen = gguf_model(path, KW, w, "llama", orc.FMT_Q8_0)
    cfg, wdir, _ = E.gguf_prepare(path, str(tmp_path / "prepared"), emit_dequantized_blobs=True)
    n, vals = E.blob_weight_load(os.path.join(wdir, "layers/1/wk.bin"))
    assert n == seen["layers"][1]["wk"].size
    assert np.array_equal(vals, seen["layers"][1]["wk"].ravel().astype(np.float16).astype(np.float32))   # half-split row order


def test_gguf_errors(E, tmp_path):
    import espresso_amd._lib as lib
    bad = tmp_path / "bad.gguf"
    bad.write_bytes(b"GGML" + b"\0" * 64)
    with pytest.raises(lib.EspressoError, match="bad magic"):
        E.gguf_prepare(str(bad), str(tmp_path / "o1"))
    import struct
    bad.write_bytes(struct.pack("<IIQQ", 0x46554747, 1, 0, 0))
    with pytest.raises(lib.EspressoError, match="unsupported GGUF version"):
        E.gguf_prepare(str(bad), str(tmp_path / "o2"))
    write_gguf(str(bad), {"general.architecture": "bert"}, [])
    with pytest.raises(lib.EspressoError, match="unsupported architecture"):
        E.gguf_prepare(str(bad), str(tmp_path / "o3"))
    w = mu.random_weights(orc.LlamaConfig(**KW), 63, std=0.08)
    good = str(tmp_path / "g.gguf")
    gguf_model(good, KW, w, "llama", orc.FMT_Q8_0)
    data = open(good, "rb").read()
    bad.write_bytes(data[:len(data) // 2])                                              # tensor data cut short
    with pytest.raises(lib.EspressoError, match="past the end"):
        E.gguf_prepare(str(bad), str(tmp_path / "o4"))


def test_harness_with_gpu_models(E, tmp_path):
    import espresso_amd.llama as ll
    full_kw, draft_kw = dict(KW, n_layer=3), dict(KW, n_layer=1)
    rts = []
    for kw, seed in ((full_kw, 71), (draft_kw, 72)):
        packed, _ = mu.pack_weights(mu.random_weights(orc.LlamaConfig(**kw), seed, std=0.08), orc.FMT_Q8_0)
        rt = ll.LlamaRuntime(ll.MultiModelConfig(**kw))
        ll.load_packed_weights(rt, packed, orc.FMT_Q8_0)
        rts.append(rt)
    plain, _ = rts[0].generate(PROMPT, 24)
    toks, com, acc = E.harness_generate(PROMPT, 23, target=rts[0], draft=rts[1])
    assert toks[:23] == plain[:23] and len(toks) in (23, 24)
    assert all(c in (1, 2) for c in com) and all(a == c - 1 for a, c in zip(acc, com)) and sum(com) == len(toks)
    # LocalBigramArtifactBuilder golden: [35] -> [105, 110, 116, 32], committed [2, 2], accepted [1, 1]
    from test_oracle_runtime import bigram_model
    _, w = bigram_model(d_model=128, vocab=128)
    packed, _ = mu.pack_weights(w, orc.FMT_F16)
    kw = dict(n_layer=1, n_head=2, n_kv_head=2, d_model=128, head_dim=64, hidden_dim=16, vocab=128, max_seq=32)
    pair = []
    for _ in range(2):
        rt = ll.LlamaRuntime(ll.MultiModelConfig(**kw))
        ll.load_packed_weights(rt, packed, orc.FMT_F16)
        pair.append(rt)
    toks, com, acc = E.harness_generate([35], 4, target=pair[0], draft=pair[1])
    assert toks == [105, 110, 116, 32] and com == [2, 2] and acc == [1, 1]


def test_engine_temperature_sampling_replays_on_the_oracle(E, tmp_path):
    """generate(temperature > 0): every step reads the GPU's logits back and applies sampleToken
    (RealModelInferenceEngine.swift:8036-8081) with SplitMix64 draws.  Replayed here: the oracle runtime is advanced with
    the engine's tokens and must choose the same token from its own logits whenever the draw is not within the logit
    tolerance of a bucket edge; the stream is reproducible per seed and differs between seeds."""
    w = mu.random_weights(orc.LlamaConfig(**KW), 43, std=0.08, norm_jitter=0.05)
    seen = write_weight_dir(str(tmp_path), KW, w)
    e = E.RealModelInferenceEngine(gpu_cfg(KW), str(tmp_path))
    env = {"ESPRESSO_HIP_SAMPLING_SEED": "12345"}
    toks, res = e.generate(PROMPT, 24, temperature=0.8, environment=env)
    assert len(toks) == 24 and res["exact_head_backend"] == "hip_gemv_logits_host_sampling"
    assert e.generate(PROMPT, 24, temperature=0.8, environment=env)[0] == toks
    assert e.generate(PROMPT, 24, temperature=0.8, environment={"ESPRESSO_HIP_SAMPLING_SEED": "999"})[0] != toks
    units = E.splitmix64_units(12345, 24)
    o = mu.load_oracle(orc.LlamaConfig(gemv_inputs_fp16=True, **KW), seen)
    o.prefill(PROMPT)
    agree = 0
    for t, u in zip(toks, units):
        lo = o.logits()
        mine = orc.sample_token(lo, 0.8, u)
        # the same draw a hair to either side: if all three agree the choice is insensitive to the logit tolerance
        stable = mine == orc.sample_token(lo, 0.8, min(u + 5e-4, 0.999999)) == orc.sample_token(lo, 0.8, max(u - 5e-4, 0.0))
        if stable:
            assert mine == t
            agree += 1
        o.advance(t)
    assert agree >= 12
    e.close()


def test_engine_generates_from_prompt_text(E, tmp_path):
    """generate(prompt:maxTokens:temperature:) (:1405-1437): the tokenizer found in tokenizerDir encodes the prompt,
    the token-id path runs, and the text is the decoded prompt + generated tokens."""
    import struct

    import espresso_amd._lib as lib
    import espresso_amd.tokenizer as T
    w = mu.random_weights(orc.LlamaConfig(**KW), 47, std=0.08, norm_jitter=0.05)
    weights = tmp_path / "weights"
    seen = write_weight_dir(str(weights), KW, w)
    # a byte-fallback SentencePiece vocabulary of the model's size: "▁", 26 letters, word pieces, then <0xNN> bytes
    pieces = [("▁", 0.0)] + [(chr(97 + i), 0.0) for i in range(26)] + [("▁a", 1.0), ("▁ab", 2.0), ("bc", 1.5), ("▁the", 3.0), ("th", 1.0), ("▁th", 2.0)]
    pieces += [(f"<0x{b:02X}>", 0.0) for b in range(256)]
    pieces += [(f"zz{i}", 0.0) for i in range(KW["vocab"] - len(pieces))]
    tok_dir = tmp_path / "tok"
    tok_dir.mkdir()
    data = struct.pack("<i", 16)
    for piece, score in pieces:
        raw = piece.encode()
        data += struct.pack("<fi", score, len(raw)) + raw
    (tok_dir / "tokenizer.model").write_bytes(data)
    tok = T.Tokenizer.from_dir(gpu_cfg(KW), str(tok_dir))
    prompt = "the abc é"
    prompt_ids = tok.encode(prompt)
    assert tok.decode(prompt_ids) == prompt

    e = E.RealModelInferenceEngine(gpu_cfg(KW), str(weights), tokenizer_dir=str(tok_dir))
    text, toks, res = e.generate_text(prompt, 12)
    assert toks == oracle_tokens(KW, seen, prompt_ids, 12)                     # same ids as the token-id entry point
    assert toks == e.generate(prompt_ids, 12)[0]
    assert text == tok.decode(prompt_ids + toks)
    assert res["token_count"] == 12
    # nothing to generate: the prompt decoded back (:1427-1437)
    text0, toks0, _ = e.generate_text(prompt, 0)
    assert (text0, toks0) == (prompt, [])
    e.close()
    # a prompt that encodes to nothing is refused (encodePrompt, :5404-5408): byte-level BPE of the empty string
    bpe_dir = tmp_path / "bpe"
    bpe_dir.mkdir()
    (bpe_dir / "vocab.json").write_text(json.dumps({chr(33 + i): i for i in range(8)}))
    (bpe_dir / "merges.txt").write_text("#version: 0.2\n")
    e = E.RealModelInferenceEngine(gpu_cfg(KW), str(weights), tokenizer_dir=str(bpe_dir))
    with pytest.raises(lib.EspressoError, match="no tokens"):
        e.generate_text("", 4)
    assert e.generate_text("!#", 3)[0].startswith("!#")
    e.close()
    # an engine without a tokenizer directory has the token-id entry points only
    e = E.RealModelInferenceEngine(gpu_cfg(KW), str(weights))
    with pytest.raises(lib.EspressoError, match="without a tokenizer"):
        e.generate_text(prompt, 4)
    e.close()
    # a tokenizer directory that holds none of the candidates fails the build, as loadTokenizer throws (:7609-7611)
    empty = tmp_path / "empty"
    empty.mkdir()
    with pytest.raises(lib.EspressoError, match="missing path"):
        E.RealModelInferenceEngine(gpu_cfg(KW), str(weights), tokenizer_dir=str(empty))


def test_bundle_selects_the_exact_two_token_path(E, tmp_path):
    """ESPRuntimeRunner.generate (ESPBundledRuntime.swift:49-80): the bundle's [draft] section reaches the engine as
    ESPRESSO_BUNDLE_DRAFT_* and the text comes from the bundle's tokenizer."""
    import struct

    import espresso_amd.bundle as B
    import espresso_amd.tokenizer as T
    root = tmp_path / "model.esp"
    for entry in B.REQUIRED_TOP_LEVEL_ENTRIES:
        os.makedirs(root / entry)
    full_kw, draft_kw = dict(KW, n_layer=3), dict(KW, n_layer=1)
    # the stream is compared token for token: a seed for which the oracle's top-2 margin is at least 0.1 at each of the 20 steps
    # (most seeds have a step below 1e-2, which the fp16 rounding of an activation can flip)
    seen_f = write_weight_dir(str(root / "weights"), full_kw, mu.random_weights(orc.LlamaConfig(**full_kw), 80, std=0.08))
    seen_d = write_weight_dir(str(root / "weights" / "draft"), draft_kw, mu.random_weights(orc.LlamaConfig(**draft_kw), 62, std=0.08))
    (root / "weights" / "draft.json").write_text(json.dumps({"model_dir": "draft", "tokenizer_dir": None, "model_id": "d"}))
    pieces = [("▁", 0.0)] + [(chr(97 + i), 0.0) for i in range(26)] + [("▁the", 2.0), ("▁t", 1.0), ("▁th", 1.5)] + [(f"<0x{b:02X}>", 0.0) for b in range(256)]
    pieces += [(f"zz{i}", 0.0) for i in range(KW["vocab"] - len(pieces))]
    data = struct.pack("<i", 16)
    for piece, score in pieces:
        raw = piece.encode()
        data += struct.pack("<fi", score, len(raw)) + raw
    (root / "tokenizer" / "tokenizer.model").write_bytes(data)

    def manifest(draft_class="exact", target=40):
        return f"""format_version = "1.1.0"
model_id = "tiny.llama"
model_family = "llama"
architecture_version = "decoder-v1"
tokenizer_contract = "sentencepiece-v1"
supported_backends = ["ane-private", "cpu-safe"]
supported_profiles = ["prefill_256", "decode_1"]
max_context = {KW['max_seq']}
context_target_tokens = {target}
adapter_slots = 0
accuracy_baseline_ref = "benchmarks/accuracy.json"
performance_baseline_ref = "benchmarks/perf.json"
signature_ref = "signatures/content-hashes.json"
[compression_policy]
name = "fp16"
weight_bits = 16
[draft]
kind = "exact_two_token"
behavior_class = "{draft_class}"
horizon = 2
verifier = "exact"
rollback = "exact_replay"
artifact_ref = "weights/draft.json"
acceptance_metric = "accepted_future_tokens"
"""
    (root / "manifest.toml").write_text(manifest())
    B.write_signature_catalog(str(root))
    b = B.RuntimeBundle(str(root))
    prompt = "the cat"
    ids = T.Tokenizer.from_dir(gpu_cfg(full_kw), str(root / "tokenizer")).encode(prompt)
    text, toks, res, sel = b.generate(prompt, 20)
    of = mu.load_oracle(orc.LlamaConfig(gemv_inputs_fp16=True, **full_kw), seen_f)
    od = mu.load_oracle(orc.LlamaConfig(gemv_inputs_fp16=True, **draft_kw), seen_d)
    want, st = orc.generate_two_token(of, od, ids, 20)
    assert toks == want
    assert res["exact_head_backend"] == "hip_exact_two_token_draft" and res["has_two_token_stats"] == 1
    assert res["accepted_future_tokens_per_pass"] == pytest.approx(st["accepted_total"] / st["passes"])
    assert sel["backend"] == "ane-private" and sel["has_draft"]
    assert text.startswith(prompt)
    # host without the private backend: the other backend, the same engine, the same tokens
    assert b.generate(prompt, 20, environment={"ESPRESSO_DISABLE_ANE_PRIVATE": "1"})[3]["backend"] == "cpu-safe"
    # prompt + maxTokens beyond the bundle's context target is refused before the model is built (ESPRuntimeResolverTests.swift:267-326)
    with pytest.raises(B.BundleError) as e:
        b.generate(prompt, 40)
    assert (e.value.case, e.value.detail, e.value.detail2) == ("requestedContextExceedsTarget", len(ids) + 40, 40)
    b.close()
    # an approximate draft is not passed on: plain greedy
    (root / "manifest.toml").write_text(manifest(draft_class="approximate"))
    text2, toks2, res2, _ = B.RuntimeBundle(str(root), verify_signatures=False).generate(prompt, 20)
    assert res2["exact_head_backend"] == "hip_gemv_argmax" and toks2 == toks and text2 == text


def test_run_gguf_front_door(E, tmp_path):
    """RunGGUF.main (RunGGUF.swift:68-113): prepare through the artifact cache, build with the tokenizer directory,
    generate from the prompt text, clean up what is not a managed cache entry."""
    import struct
    import subprocess
    import sys

    import espresso_amd.tokenizer as T
    w = mu.random_weights(orc.LlamaConfig(**KW), 71, std=0.08, norm_jitter=0.05)
    path = str(tmp_path / "m.gguf")
    seen = gguf_model(path, KW, w, "llama", orc.FMT_Q8_0)
    pieces = [("▁", 0.0)] + [(chr(97 + i), 0.0) for i in range(26)] + [("▁the", 3.0), ("th", 1.0), ("▁th", 2.0)] + [(f"<0x{b:02X}>", 0.0) for b in range(256)]
    pieces += [(f"zz{i}", 0.0) for i in range(KW["vocab"] - len(pieces))]
    tok_dir = tmp_path / "tok"
    tok_dir.mkdir()
    data = struct.pack("<i", 16)
    for piece, score in pieces:
        raw = piece.encode()
        data += struct.pack("<fi", score, len(raw)) + raw
    (tok_dir / "tokenizer.model").write_bytes(data)
    tok = T.Tokenizer.from_dir(gpu_cfg(KW), str(tok_dir))
    prompt = "the cat"
    ids = tok.encode(prompt)
    want = oracle_tokens(dict(KW, eos_token=2), seen, ids, 10)

    cache = tmp_path / "cache"
    env = {"ESPRESSO_GGUF_PREPARE_CACHE_ROOT": str(cache)}
    r = E.run_gguf(path, str(tok_dir), prompt, 10, env)
    assert r["tokens"] == want and r["text"] == tok.decode(ids + want)
    assert r["tensor_count"] == 3 + 9 * KW["n_layer"] and r["config"].d_model == KW["d_model"]
    assert r["kept_weight_dir"] and os.path.dirname(r["weight_dir"]) == str(cache)      # a managed cache entry survives cleanup
    again = E.run_gguf(path, str(tok_dir), prompt, 10, env)
    assert again["weight_dir"] == r["weight_dir"] and again["tokens"] == want
    # cache off: a temporary directory, removed unless ESPRESSO_GGUF_KEEP_WEIGHT_DIR=1
    off = E.run_gguf(path, str(tok_dir), prompt, 4, {"ESPRESSO_GGUF_PREPARE_CACHE": "0"})
    assert off["tokens"] == want[:4] and not off["kept_weight_dir"] and not os.path.exists(off["weight_dir"])
    kept = E.run_gguf(path, str(tok_dir), prompt, 4, {"ESPRESSO_GGUF_FORCE_FRESH_PREPARE": "1", "ESPRESSO_GGUF_KEEP_WEIGHT_DIR": "1"})
    assert kept["kept_weight_dir"] and os.path.exists(os.path.join(kept["weight_dir"], "metadata.json"))
    E.gguf_cleanup(kept["weight_dir"])
    # a missing tokenizer fails the build and still cleans up
    import espresso_amd._lib as lib
    with pytest.raises(lib.EspressoError):
        E.run_gguf(path, str(tmp_path / "no-tokenizer"), prompt, 4, {"ESPRESSO_GGUF_PREPARE_CACHE": "0"})
    # the runner's command line: text on stdout, the report on stderr, exit status 1 with usage when arguments are missing
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    run = subprocess.run([sys.executable, "-m", "espresso_amd.run_gguf", path, str(tok_dir), prompt, "10"], cwd=root, capture_output=True, text=True,
                         env=dict(os.environ, **env), timeout=300)
    assert run.returncode == 0, run.stderr
    assert run.stdout.rstrip("\n") == r["text"]
    assert "Tokens generated: 10" in run.stderr and "Prepared: llama, 2 layers" in run.stderr
    short = subprocess.run([sys.executable, "-m", "espresso_amd.run_gguf", path], cwd=root, capture_output=True, text=True, timeout=120)
    assert short.returncode == 1 and "Usage" in short.stderr
