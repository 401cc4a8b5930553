"""Host-side pieces of the boundary that need no GPU: exported symbols, BLOBFILE, paths, metadata,
the promotion plan and the exact two-token harness driven by scripted models (the reference's own
test doubles, Tests/EspressoTests/GenerationHarnessTests.swift:63-270, 482-619)."""
import ctypes as C
import os
import re

import numpy as np
import pytest

import espresso_amd._lib as lib
import espresso_amd.engine as eng
import espresso_amd.llama as ll
from oracle import oracle as orc

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_library_exports_every_declared_symbol():
    names = set()
    for name in ("espresso_hip.h", "espresso_hip_bench.h"):
        header = open(os.path.join(ROOT, "include", name)).read()
        header = re.sub(r"/\*.*?\*/", "", header, flags=re.S)
        found = set(re.findall(r"\b(esp_[a-z0-9_]+)\s*\(", header))
        assert len(found) > (40 if name == "espresso_hip.h" else 5)
        names |= found
    L = lib.load_library()
    missing = [n for n in sorted(names) if not hasattr(L, n)]
    assert not missing, missing


def test_headers_are_plain_c11_and_the_boundary_header_holds_no_measurement_calls():
    """The module map hands espresso_hip.h to a C importer (Swift's clang importer reads it as C): it has to stay valid
    C11 with no C++ or compiler extensions.  Measurement and tuning calls live in espresso_hip_bench.h, outside the
    drop-in boundary."""
    import shutil
    import subprocess
    cc = shutil.which("gcc") or shutil.which("cc")
    if cc is None:
        pytest.skip("no C compiler")
    inc = os.path.join(ROOT, "include")
    for name in ("espresso_hip.h", "espresso_hip_bench.h"):
        proc = subprocess.run([cc, "-x", "c", "-std=c11", "-pedantic", "-Wall", "-Wextra", "-Werror", "-fsyntax-only", "-I", inc,
                               os.path.join(inc, name)], capture_output=True, text=True)
        assert proc.returncode == 0, proc.stderr
    boundary = open(os.path.join(inc, "espresso_hip.h")).read()
    for name in ("esp_gemv_time", "esp_gemv_stamps", "esp_set_tuning", "esp_hbm_read_probe", "esp_llama_time_kernel",
                 "esp_llama_set_kernel_timing", "esp_llama_kernel_times"):
        assert name + "(" not in boundary, name
    modulemap = open(os.path.join(inc, "module.modulemap")).read()
    assert 'header "espresso_hip.h"' in modulemap and "espresso_hip_bench.h" not in modulemap


def test_no_device_fails_loudly_without_cpu_fallback():
    if os.path.exists("/dev/kfd"):
        pytest.skip("GPU present")
    import espresso_amd.ops as ops
    with pytest.raises(lib.EspressoError, match="no CPU fallback"):
        ops.init()
    with pytest.raises(lib.EspressoError):
        ops.dequantize(orc.FMT_Q8_0, np.zeros(34, np.uint8), 32)


def test_weight_blob_matches_reference_layout_and_oracle(tmp_path):
    w = np.random.default_rng(0).normal(0, 0.02, 1000).astype(np.float32)
    w[:6] = [0.0, -0.0, 65504.0, 1e-8, 6.1e-5, 1.0 + 2 ** -11]
    blob = eng.weight_blob_build(w)
    assert blob == orc.blob_build(w)
    assert blob[0] == 1 and blob[4] == 2 and blob[64:68] == bytes([0xEF, 0xBE, 0xAD, 0xDE]) and blob[68] == 1
    assert int.from_bytes(blob[72:76], "little") == 2000 and int.from_bytes(blob[80:84], "little") == 128
    p = tmp_path / "w.bin"
    p.write_bytes(blob)
    n, back = eng.blob_weight_load(str(p))
    assert n == 1000 and np.array_equal(back, w.astype(np.float16).astype(np.float32))
    # BlobWeightLoaderError cases (Sources/ModelSupport/BlobWeightLoader.swift:3-9, 62-90)
    cases = {-1: blob[:100], -2: blob[:64] + b"\0" + blob[65:], -3: blob[:80] + bytes([64]) + blob[81:], -4: blob[:-2],
             -5: blob[:72] + bytes([7]) + blob[73:]}
    for code, data in cases.items():
        p.write_bytes(data)
        assert eng.blob_weight_load(str(p))[0] == code
    assert eng.blob_weight_load(str(tmp_path / "missing.bin"))[0] == -6
    p.write_bytes(eng.weight_blob_build(np.zeros(0, np.float32)))
    assert eng.blob_weight_load(str(p))[0] == 0                                  # empty payload


def test_layer_weight_paths():
    names = {ll.SLOT_RMS_ATT: "rms_att", ll.SLOT_WQ: "wq", ll.SLOT_WK: "wk", ll.SLOT_WV: "wv", ll.SLOT_WO: "wo",
             ll.SLOT_RMS_FFN: "rms_ffn", ll.SLOT_W1: "w1", ll.SLOT_W2: "w2", ll.SLOT_W3: "w3", ll.SLOT_Q_NORM: "q_norm",
             ll.SLOT_K_NORM: "k_norm"}
    for slot, name in names.items():
        assert eng.layer_weight_path(3, "/tmp/weights", slot) == f"/tmp/weights/layers/3/{name}.bin"
    with pytest.raises(lib.EspressoError):
        eng.layer_weight_path(0, "/tmp/weights", ll.SLOT_LM_HEAD)


def test_metadata_round_trip_and_reference_keys(tmp_path):
    cfg = ll.MultiModelConfig(n_layer=6, n_head=12, n_kv_head=4, d_model=768, head_dim=64, hidden_dim=2048, vocab=32000, max_seq=256,
                              norm_eps=1e-6, rope_theta=500000.0, eos_token=2, name="llama")
    path = str(tmp_path / "metadata.json")
    eng.write_metadata(cfg, path)
    import json
    raw = json.load(open(path))
    assert set(raw) == {"name", "nLayer", "nHead", "nKVHead", "dModel", "headDim", "hiddenDim", "vocab", "maxSeq", "normEps",
                        "ropeTheta", "architecture", "eosToken"}
    assert raw["architecture"] == "llama" and raw["nKVHead"] == 4 and raw["eosToken"] == 2
    back = eng.load_metadata(path)
    assert np.float32(back.norm_eps) == np.float32(cfg.norm_eps)      # normEps is a Float in the reference
    back.norm_eps = cfg.norm_eps
    assert back == cfg
    # a file written by other tooling: extra keys, nested values, no eosToken
    open(path, "w").write('{"nLayer": 1, "nHead": 2, "nKVHead": 1, "dModel": 8, "headDim": 4, "hiddenDim": 16, "vocab": 32, '
                          '"maxSeq": 16, "architecture": "llama", "extra": {"a": [1, 2, {"b": null}]}, "name": "tiny\\u002dllama"}')
    t = eng.load_metadata(path)
    assert (t.n_layer, t.vocab, t.eos_token, t.name) == (1, 32, -1, "tiny-llama")
    open(path, "w").write('{"nLayer": 1')
    with pytest.raises(lib.EspressoError, match="not valid JSON"):
        eng.load_metadata(path)
    open(path, "w").write('{"nLayer": 1}')
    with pytest.raises(lib.EspressoError, match="missing nHead"):
        eng.load_metadata(path)


def test_promotion_plan():
    """GenerationHarnessTests.swift:589-619"""
    a = eng.promotion_plan(5, 6, 6, 7, 2)
    assert a == {"committed_tokens": [5, 6], "next_current_token": 7, "committed_exact_token_count": 2,
                 "accepted_future_token_count": 1, "promoted_step_count": 2}
    r = eng.promotion_plan(5, 9, 6, 7, 2)
    assert r == {"committed_tokens": [5], "next_current_token": 6, "committed_exact_token_count": 1,
                 "accepted_future_token_count": 0, "promoted_step_count": 1}
    assert eng.promotion_plan(5, 6, 6, 7, 1)["committed_tokens"] == [5]          # budget 1 never commits two


class FakeExactTwoTokenModel:
    """FakeExactTwoTokenModel: a scripted queue of pass results (GenerationHarnessTests.swift:200-270)."""

    def __init__(self, selected_prefill_token, passes):
        self.selected, self.queue = selected_prefill_token, list(passes)
        self.reset_count, self.prefill_calls, self.pass_calls = 0, [], []
        self._keep = (eng.RESET_FN(self._reset), eng.PREFILL_FN(self._prefill), eng.PASS_FN(self._pass))
        self.struct = eng.ExactTwoTokenModelStruct(None, *self._keep)

    def _reset(self, ctx):
        self.reset_count += 1
        return 0

    def _prefill(self, ctx, toks, n, out):
        self.prefill_calls.append([toks[i] for i in range(n)])
        out[0] = self.selected
        return 0

    def _pass(self, ctx, current, budget, res):
        self.pass_calls.append((current, budget))
        if not self.queue:
            return 1
        committed, nxt, advance_ms, accepted, count = self.queue.pop(0)
        r = res.contents
        for i, t in enumerate(committed[:2]):
            r.committed_tokens[i] = t
        r.committed_count = len(committed)
        r.next_current_token = nxt
        r.state_advance_latency_ms = advance_ms
        r.accepted_future_token_count = accepted
        r.committed_exact_token_count = count
        return 0


def test_harness_tracks_pass_metrics_and_future_acceptance():
    """GenerationHarnessTests.swift:482-535: trace [5,6,7], accepted [1,0], committed [2,1]."""
    m = FakeExactTwoTokenModel(5, [([5, 6], 7, 1.15, 1, 2), ([7], 8, 0.0, 0, 1)])
    toks, com, acc = eng.harness_generate([9], 3, model=m.struct)
    assert toks == [5, 6, 7] and acc == [1, 0] and com == [2, 1]
    assert m.reset_count == 1 and m.prefill_calls == [[9]] and m.pass_calls == [(5, 3), (7, 1)]
    assert sum(com) / len(com) == 1.5 and sum(acc) / len(acc) == 0.5


def test_harness_future_rejection():
    """GenerationHarnessTests.swift:537-587"""
    m = FakeExactTwoTokenModel(2, [([2], 4, 0.0, 0, 1), ([4], 6, 0.0, 0, 1)])
    toks, com, acc = eng.harness_generate([1], 2, model=m.struct)
    assert toks == [2, 4] and acc == [0, 0] and com == [1, 1]


@pytest.mark.parametrize("passes,message", [
    ([([], 1, 0.0, 0, 0)], "must commit at least one token"),
    ([([9, 6], 7, 1.0, 1, 2)], "must commit current token first"),
    ([([5, 6], 7, 1.0, 1, 2)], "with remaining budget 1"),                      # budget 1, two committed
    ([([5, 6, 7], 8, 0.0, 0, 3)], "committed 3 tokens"),
    ([([5], 6, 0.0, 2, 1)], "must be in 0...1"),
    ([([5, 6], 7, 0.0, 0, 1)], "must equal committed token count"),
    ([([5], 6, 1.0, 1, 1)], "requires exactly two committed tokens"),
    ([([5], 6, 0.5, 0, 1)], "must be zero when no future token is accepted"),
])
def test_harness_rejects_invariant_violations(passes, message):
    """The guards of ExactTwoTokenGenerationHarness.generate (GenerationHarness.swift:640-672)."""
    budget = 1 if "budget 1" in message else 4
    m = FakeExactTwoTokenModel(5, passes)
    with pytest.raises(lib.EspressoError, match=re.escape(message)):
        eng.harness_generate([9], budget, model=m.struct)


def test_harness_argument_errors():
    m = FakeExactTwoTokenModel(5, [])
    with pytest.raises(lib.EspressoError, match="promptTokens must not be empty"):
        eng.harness_generate([], 3, model=m.struct)
    with pytest.raises(lib.EspressoError, match="maxNewTokens must be > 0"):
        eng.harness_generate([1], 0, model=m.struct)
    with pytest.raises(lib.EspressoError, match="callback"):
        eng.harness_generate([1], 2, model=m.struct)                             # the scripted queue is empty


def test_sample_token_follows_reference_rule():
    """sampleToken (RealModelInferenceEngine.swift:8036-8068): host code of the library and the oracle against the rule
    restated with numpy cumulative sums."""
    rng = np.random.default_rng(12)
    logits = rng.normal(0, 2, 1000).astype(np.float32)
    assert eng.sample_token(logits, 0.0, 0.3) == orc.sample_token(logits, 0.0, 0.3) == int(np.argmax(logits))
    tie = np.array([1, 5, 5, 2], np.float32)
    assert eng.sample_token(tie, 0.0, 0.9) == 1                                  # first maximum
    for temperature in (0.5, 1.0, 2.0):
        w = np.exp(((logits - logits.max()) / np.float32(temperature)).astype(np.float64))
        cum = np.cumsum(w)
        for unit in (0.0, 1e-12, 0.1, 0.5, 0.9, 0.999999):
            want = int(np.searchsorted(cum, unit * cum[-1], side="left"))
            got = eng.sample_token(logits, temperature, unit)
            assert got == orc.sample_token(logits, temperature, unit)
            assert abs(got - want) <= 1                                           # running subtraction vs prefix sums: last-ulp ties
    # degenerate totals fall back to the first maximum
    assert eng.sample_token(np.array([0, np.inf, 1], np.float32), 1.0, 0.5) == 1
    # SplitMix64 unit doubles: in [0, 1), reproducible, first value of seed 0 known in closed form
    u = eng.splitmix64_units(0, 4)
    assert u == eng.splitmix64_units(0, 4) and all(0.0 <= v < 1.0 for v in u)
    assert u[0] == (0xE220A8397B1DCDAF >> 11) * 2.0 ** -53                      # SplitMix64(0).next() = 0xE220A8397B1DCDAF
    # empirical distribution over many draws matches softmax(logits / T)
    small = np.array([0.0, 1.0, 2.0, -1.0], np.float32)
    units = eng.splitmix64_units(7, 20000)
    counts = np.bincount([eng.sample_token(small, 1.0, v) for v in units], minlength=4) / 20000
    p = np.exp(small - small.max()); p /= p.sum()
    assert np.abs(counts - p).max() < 0.015


# ---- prepared-artifact cache of the GGUF front door (Tests/EspressoGGUFTests/GGUFModelLoaderTests.swift:110-176) ----
def test_prepare_options_parse_cache_and_sidecar_controls_from_the_environment():
    o = eng.PrepareOptions.environment({
        "ESPRESSO_GGUF_PREPARE_CACHE": "0",
        "ESPRESSO_GGUF_PREPARE_CACHE_ROOT": "/tmp/espresso-cache",
        "ESPRESSO_GGUF_SIDECAR_POLICY": "selected",
        "ESPRESSO_GGUF_SELECTED_SIDECARS": "blk.27.attn_q.weight, blk.27.attn_k.weight",
    })
    assert o.artifact_cache_enabled is False
    assert o.cache_root == "/tmp/espresso-cache"
    assert o.sidecar_mode == "selected" and o.selected_sidecars == {"blk.27.attn_q.weight", "blk.27.attn_k.weight"}
    # defaults, the force-fresh switch, spellings of the policy, an unknown policy
    d = eng.PrepareOptions.environment({})
    assert d.artifact_cache_enabled and d.cache_root is None and d.sidecar_mode == "automatic" and not d.selected_sidecars
    assert not eng.PrepareOptions.environment({"ESPRESSO_GGUF_FORCE_FRESH_PREPARE": "yes", "ESPRESSO_GGUF_PREPARE_CACHE": "1"}).artifact_cache_enabled
    assert eng.PrepareOptions.environment({"ESPRESSO_GGUF_PREPARE_CACHE": " On "}).artifact_cache_enabled
    for raw, mode in (("OFF", "none"), (" none ", "none"), ("auto", "automatic"), ("Essential", "essential"), ("full", "full"), ("bogus", "automatic")):
        assert eng.PrepareOptions.environment({"ESPRESSO_GGUF_SIDECAR_POLICY": raw}).sidecar_mode == mode
    assert eng.PrepareOptions.environment({"ESPRESSO_GGUF_PREPARE_CACHE_ROOT": "   "}).cache_root is None
    assert eng.PrepareOptions.environment({"ESPRESSO_GGUF_PREPARE_CACHE_ROOT": "~/c"}).cache_root == os.path.expanduser("~/c")


def test_artifact_cache_key_tracks_prepare_options(tmp_path):
    path = tmp_path / "k.gguf"
    path.write_bytes(b"QGUF")
    essential = eng.gguf_artifact_cache_key(str(path), eng.PrepareOptions(sidecar_mode="essential"))
    assert essential == eng.gguf_artifact_cache_key(str(path), eng.PrepareOptions(sidecar_mode="essential"))
    selected = eng.gguf_artifact_cache_key(str(path), eng.PrepareOptions(sidecar_mode="selected", selected_sidecars=["blk.27.attn_q.weight"]))
    assert essential != selected and re.fullmatch(r"[0-9a-f]{64}", essential)
    # the selection, the converter's switches, the file's size and its path all enter the key; other variables do not
    assert selected != eng.gguf_artifact_cache_key(str(path), eng.PrepareOptions(sidecar_mode="selected", selected_sidecars=["blk.27.attn_k.weight"]))
    assert essential != eng.gguf_artifact_cache_key(str(path), eng.PrepareOptions(sidecar_mode="essential"), {"ESPRESSO_FORCE_QK_INVERSE_INTERLEAVE": "1"})
    assert essential == eng.gguf_artifact_cache_key(str(path), eng.PrepareOptions(sidecar_mode="essential"), {"HOME": "/elsewhere", "ESPRESSO_FORCE_QK_INVERSE_INTERLEAVE": ""})
    assert essential == eng.gguf_artifact_cache_key(str(tmp_path / "sub" / ".." / "k.gguf"), eng.PrepareOptions(sidecar_mode="essential"))
    path.write_bytes(b"QGUF+")
    assert essential != eng.gguf_artifact_cache_key(str(path), eng.PrepareOptions(sidecar_mode="essential"))
    with pytest.raises(lib.EspressoError):
        eng.gguf_artifact_cache_key(str(tmp_path / "absent.gguf"), eng.PrepareOptions())


def test_cleanup_removes_a_directory_and_keeps_managed_cache_entries(tmp_path):
    plain = tmp_path / "espresso_gguf_test"
    plain.mkdir()
    (plain / "test.bin").write_bytes(b"\x01")
    eng.gguf_cleanup(str(plain))
    assert not plain.exists()
    cached = tmp_path / "espresso_gguf_cached"
    cached.mkdir()
    (cached / ".espresso-gguf-cache-artifact").write_bytes(b"")
    eng.gguf_cleanup(str(cached))
    assert cached.exists()
    assert eng.gguf_default_cache_root().endswith(os.path.join("Espresso", "gguf-prepared"))


def test_prepare_through_the_artifact_cache(tmp_path):
    import json
    import sys
    sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
    import model_util as mu
    from gguf_writer import gguf_model
    kw = dict(n_layer=1, n_head=2, n_kv_head=1, d_model=64, head_dim=32, hidden_dim=256, vocab=256, max_seq=16)
    w = mu.random_weights(orc.LlamaConfig(**kw), 5, std=0.08)
    path = str(tmp_path / "m.gguf")
    gguf_model(path, kw, w, "llama", orc.FMT_Q8_0)
    root = tmp_path / "cache"
    opts = eng.PrepareOptions(cache_root=str(root))
    cfg, wdir, count = eng.gguf_prepare_cached(path, opts)
    key = eng.gguf_artifact_cache_key(path, opts)
    assert wdir == str(root / key) and count == 3 + 9 and cfg.d_model == 64
    manifest = json.load(open(os.path.join(wdir, "prepare-manifest.json")))
    assert manifest["tensorCount"] == count and manifest["ggufPath"] == path and manifest["sidecarMode"] == "automatic"
    assert manifest["fileSize"] == os.path.getsize(path) and manifest["version"] == 2
    assert os.path.exists(os.path.join(wdir, ".espresso-gguf-cache-artifact"))
    # a second prepare returns the cached directory untouched (a file planted in it survives), and cleanup keeps it
    open(os.path.join(wdir, "planted"), "w").close()
    cfg2, wdir2, count2 = eng.gguf_prepare_cached(path, opts)
    assert (wdir2, count2, cfg2.vocab) == (wdir, count, cfg.vocab) and os.path.exists(os.path.join(wdir, "planted"))
    eng.gguf_cleanup(wdir)
    assert os.path.isdir(wdir)
    # an entry without its metadata is rebuilt
    os.remove(os.path.join(wdir, "metadata.json"))
    _, wdir3, _ = eng.gguf_prepare_cached(path, opts)
    assert wdir3 == wdir and os.path.exists(os.path.join(wdir, "metadata.json")) and not os.path.exists(os.path.join(wdir, "planted"))
    # other options, another entry; sidecar policy "none" writes no float32 sidecar, "selected" only the named tensor
    none = eng.PrepareOptions(cache_root=str(root), sidecar_mode="none")
    _, wdir_none, _ = eng.gguf_prepare_cached(path, none)
    assert wdir_none != wdir and not os.path.exists(os.path.join(wdir_none, "rms_final.float32.bin"))
    assert os.path.exists(os.path.join(wdir, "rms_final.float32.bin"))
    sel = eng.PrepareOptions(cache_root=str(root), sidecar_mode="selected", selected_sidecars=["blk.0.attn_norm.weight"])
    _, wdir_sel, _ = eng.gguf_prepare_cached(path, sel)
    assert os.path.exists(os.path.join(wdir_sel, "layers/0/rms_att.float32.bin")) and not os.path.exists(os.path.join(wdir_sel, "rms_final.float32.bin"))
    # cache off: a fresh temporary directory each time, no marker, removed by cleanup
    off = eng.PrepareOptions(artifact_cache_enabled=False)
    _, t1, _ = eng.gguf_prepare_cached(path, off)
    _, t2, _ = eng.gguf_prepare_cached(path, off)
    assert t1 != t2 and os.path.basename(t1).startswith("espresso_gguf_") and not os.path.exists(os.path.join(t1, ".espresso-gguf-cache-artifact"))
    eng.gguf_cleanup(t1); eng.gguf_cleanup(t2)
    assert not os.path.exists(t1) and not os.path.exists(t2)
    # a file that is no GGUF container leaves no directory behind
    bad = tmp_path / "bad.gguf"
    bad.write_bytes(b"QGUF")
    with pytest.raises(lib.EspressoError):
        eng.gguf_prepare_cached(str(bad), opts)
    assert not os.path.exists(str(root / eng.gguf_artifact_cache_key(str(bad), opts)))


def test_cache_key_tracks_the_converter_options_and_malformed_tensors_are_refused(tmp_path):
    import sys
    sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
    import model_util as mu
    from gguf_writer import gguf_model
    kw = dict(n_layer=1, n_head=2, n_kv_head=1, d_model=64, head_dim=32, hidden_dim=256, vocab=256, max_seq=16)
    w = mu.random_weights(orc.LlamaConfig(**kw), 5, std=0.08)
    path = str(tmp_path / "m.gguf")
    gguf_model(path, kw, w, "llama", orc.FMT_Q8_0)
    opts = eng.PrepareOptions(cache_root=str(tmp_path / "cache"))
    # the same file prepared with the Q/K rows re-ordered and as stored: two cache entries, different wq bytes
    _, undone, _ = eng.gguf_prepare_cached(path, opts, qk_layout=1)
    _, stored, _ = eng.gguf_prepare_cached(path, opts, qk_layout=0)
    assert undone != stored
    wq = [open(os.path.join(d, "layers/0/wq.q8_0.bin"), "rb").read() for d in (undone, stored)]
    assert len(wq[0]) == len(wq[1]) and wq[0] != wq[1]
    assert open(os.path.join(undone, "layers/0/wv.q8_0.bin"), "rb").read() == open(os.path.join(stored, "layers/0/wv.q8_0.bin"), "rb").read()
    # the converter switch of the environment forces the re-order (same bytes as qk_layout=1, an entry of its own)
    _, forced, _ = eng.gguf_prepare_cached(path, opts, {"ESPRESSO_FORCE_QK_INVERSE_INTERLEAVE": "1"}, qk_layout=-1)
    assert forced not in (undone, stored)
    assert open(os.path.join(forced, "layers/0/wq.q8_0.bin"), "rb").read() == wq[0]
    # so does the sidecar switch (the dequantised-blob switch needs the GPU and is covered by the engine tests)
    _, bare, _ = eng.gguf_prepare_cached(path, opts, emit_float32_sidecars=False, qk_layout=1)
    assert bare != undone and not os.path.exists(os.path.join(bare, "rms_final.float32.bin"))

    # malformed files: an attn_q with the wrong number of rows, a zero dimension, an offset that wraps 64 bits
    def reshape_q(shape):
        def go(tensors):
            return [(n, t, shape if n == "blk.0.attn_q.weight" else s, raw) for n, t, s, raw in tensors]
        return go
    for i, shape in enumerate([(32, 64), (64, 32), (0, 64), (2 ** 62, 2 ** 62)]):
        bad = str(tmp_path / f"bad{i}.gguf")
        gguf_model(bad, kw, w, "llama", orc.FMT_Q8_0, mutate=reshape_q(shape))
        with pytest.raises(lib.EspressoError, match="shape"):
            eng.gguf_prepare(bad, str(tmp_path / f"out{i}"))
    far = str(tmp_path / "far.gguf")
    gguf_model(far, kw, w, "llama", orc.FMT_Q8_0, mutate=lambda ts: [t + (2 ** 64 - 64,) if t[0] == "blk.0.ffn_up.weight" else t for t in ts])
    with pytest.raises(lib.EspressoError, match="past the end"):
        eng.gguf_prepare(far, str(tmp_path / "out_far"))


# ---- ModelRegistry (Tests/ModelSupportTests/ModelConfigTests.swift:5-52) and ClassifierStrategy.select
# (Tests/RealModelInferenceTests/ClassifierStrategyTests.swift:6-148) ----
def test_model_registry_matches_the_reference_table():
    reg = eng.model_registry()
    assert len(reg) == 7 and list(reg) == sorted(reg)
    gpt2, stories = eng.model_registry_config("gpt2_124m"), eng.model_registry_config("stories110m")
    assert (gpt2.vocab, gpt2.hidden_dim, gpt2.architecture) == (50257, 3072, "gpt2")
    assert (stories.vocab, stories.hidden_dim, stories.architecture) == (32000, 2048, "llama")
    assert reg["smolLM_135m"].n_kv_head == 3 and reg["tinyLlama_1_1b"].n_head == 32 and reg["llama3_2_1b_ctx512"].max_seq == 512
    c = reg["llama3_2_1b"]
    assert (c.n_layer, c.n_head, c.n_kv_head, c.d_model, c.head_dim, c.hidden_dim, c.vocab, c.max_seq) == (16, 32, 8, 2048, 64, 8192, 128256, 2048)
    assert c.d_model == c.n_head * c.head_dim and c.rope_theta == 500000.0 and c.eos_token == 128001
    c = reg["llama3_2_3b"]
    assert (c.n_layer, c.n_head, c.n_kv_head, c.d_model, c.head_dim, c.hidden_dim, c.vocab, c.max_seq) == (28, 24, 8, 3072, 128, 8192, 128256, 2048)
    assert c.d_model == c.n_head * c.head_dim
    assert reg["stories110m"].eos_token == -1 and reg["stories110m"].rope_theta == 10000.0
    assert eng.model_registry_config("no-such-model") is None


def _cfg(name, d_model, vocab, architecture="llama"):
    return ll.MultiModelConfig(n_layer=1, n_head=1, n_kv_head=1, d_model=d_model, head_dim=64, hidden_dim=128, vocab=vocab, max_seq=32,
                               name=name, architecture=architecture)


def test_classifier_strategy_selection():
    S = eng.classifier_strategy
    assert S(_cfg("tiny-test", 64, 256)) == ("ane", "ane_classifier")
    assert S(_cfg("tinyllama-test", 2048, 32000)) == ("cpuFP16Tiled", "cpu_fp16_tiled")          # 65.5 M elements > 16 M
    assert S(eng.model_registry_config("stories110m"))[0] == "ane"                                 # the allowlist entry
    assert S(_cfg("llama2.c-stories110M", 768, 32000))[0] == "ane"                                 # bundle-style name
    assert S(_cfg("  Stories110M ", 768, 32000))[0] == "ane"
    assert S(_cfg("stories110m", 768, 50257, "gpt2"))[0] == "cpuPartitionedFP32"                   # the allowlist is for llama only
    assert S(_cfg("tinyllama-test", 2048, 32000), True) == ("cpuPartitionedFP32", "cpu_partitioned_fp32")
    assert S(_cfg("qwen3-0.6b-test", 1024, 151936))[0] == "cpuFP16Tiled"
    assert S(_cfg("gpt2-large-vocab", 768, 50257, "gpt2"))[0] == "cpuPartitionedFP32"
    assert S(_cfg("boundary-test", 64, 250000))[0] == "ane"                                        # exactly 16 M elements
    assert S(_cfg("boundary-plus-one", 64, 250001))[0] == "cpuFP16Tiled"
