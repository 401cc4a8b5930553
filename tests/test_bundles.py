"""The .esp bundle bridge (host code): the cases of Tests/ESPBundleTests/ESPManifestTests.swift and
Tests/ESPRuntimeTests/ESPRuntimeResolverTests.swift that need no model, with the SHA-256 catalog written once by
the library and once by hashlib."""
import hashlib
import json
import os

import pytest

from espresso_amd import bundle as B

FULL = """format_version = "1.1.0"
model_id = "espresso.llama.1b"
model_family = "llama"
architecture_version = "decoder-v1"
tokenizer_contract = "sentencepiece-v1"
supported_backends = ["ane-private", "cpu-safe"]
supported_profiles = ["prefill_256", "prefill_2048", "decode_1"]
max_context = 2048
context_target_tokens = 1024
model_tier = "optimized"
behavior_class = "near_exact"
adapter_slots = 4
accuracy_baseline_ref = "benchmarks/qwen-0.6b/accuracy.json"
performance_baseline_ref = "benchmarks/qwen-0.6b/perf.json"
signature_ref = "signatures/manifest.sig"
[compression_policy]
name = "int4-palettized"
weight_bits = 4
[optimization]
recipe = "stories-gqa4-distilled"
quality_gate = "short-long-prompt-parity"
teacher_model = "teacher://qwen3-0.6b"
performance_target = "110 tok/s"
[output_head]
kind = "factored"
behavior_class = "near_exact"
bottleneck = 128
groups = 1
projection_ref = "weights/cls_proj.bin"
expansion_ref = "weights/cls_expand.bin"
[draft]
kind = "exact_two_token"
behavior_class = "exact"
horizon = 2
verifier = "exact"
rollback = "exact_replay"
artifact_ref = "weights/future-sidecar.bin"
acceptance_metric = "accepted_future_tokens"
"""

LEGACY = """
    format_version = "1.0.0"
    model_id = "legacy.stories"
    model_family = "llama"
    architecture_version = "decoder-v1"
    tokenizer_contract = "sentencepiece-v1"
    supported_backends = ["ane-private", "cpu-safe"]
    supported_profiles = ["prefill_256", "decode_1"]
    max_context = 256
    adapter_slots = 0
    accuracy_baseline_ref = "benchmarks/accuracy.json"
    performance_baseline_ref = "benchmarks/perf.json"
    signature_ref = "signatures/content-hashes.json"
    [compression_policy]
    name = "native-ane-fp16"
    weight_bits = 16
"""


def edited(text, **changes):
    """Replaces `key = ...` lines (first occurrence after an optional [section] marker given as section__key)."""
    lines = text.splitlines()
    for spec, value in changes.items():
        section, _, key = spec.rpartition("__")
        active = section == ""
        for i, line in enumerate(lines):
            if line.strip().startswith("["):
                active = line.strip() == f"[{section}]"
            elif active and line.strip().startswith(key + " ="):
                if value is None:
                    lines[i] = ""
                else:
                    lines[i] = f"{key} = {value}"
                break
        else:
            raise KeyError(spec)
    return "\n".join(lines) + "\n"


# ---- ESPManifestTests.swift:5-61, :106-152 ----
def test_manifest_round_trips_and_renders_deterministically():
    rendered = B.parse_manifest(FULL)
    assert rendered == FULL                      # renderTOML's line order is the order above
    assert B.parse_manifest(rendered) == rendered
    for piece in ('model_family = "llama"', 'model_tier = "optimized"', 'behavior_class = "near_exact"', "context_target_tokens = 1024",
                  'supported_backends = ["ane-private", "cpu-safe"]', "[output_head]", 'projection_ref = "weights/cls_proj.bin"', "[draft]",
                  'artifact_ref = "weights/future-sidecar.bin"'):
        assert piece in rendered


# ---- :271-299 ----
def test_manifest_parser_backfills_defaults_for_legacy_bundles():
    rendered = B.parse_manifest(LEGACY)
    assert 'model_tier = "compat"' in rendered and 'behavior_class = "exact"' in rendered
    assert "context_target_tokens = 256" in rendered
    assert 'recipe = "legacy"' in rendered and 'quality_gate = "legacy-compatible"' in rendered
    assert "[output_head]" not in rendered and "[draft]" not in rendered


# ---- :63-88, :154-270, :301-378 and the parser's own errors (ESPBundle.swift:312-394, 700-826) ----
@pytest.mark.parametrize("text,case,payload", [
    (edited(FULL, model_id='"  "'), "emptyField", "model_id"),
    (edited(FULL, model_family='"gpt2"'), "invalidOutputHead", "output-head metadata is supported for llama bundles only"),
    (edited(FULL.replace(FULL[FULL.index("[output_head]"):FULL.index("[draft]")], ""), model_family='"qwen"'), "invalidDraft",
     "draft metadata is supported for llama bundles only"),
    (edited(FULL, draft__kind='"multi_token"'), "invalidDraft", "only exact_two_token drafts are currently supported"),
    (edited(FULL, draft__horizon="3"), "invalidDraft", "exact_two_token draft requires horizon == 2"),
    (edited(FULL, draft__horizon="1"), "invalidDraft", "draft horizon must be > 1"),
    (edited(FULL, output_head__bottleneck=None), "invalidOutputHead", "factored output head requires bottleneck > 0"),
    (edited(FULL, output_head__groups="0"), "invalidOutputHead", "factored output head requires groups > 0"),
    (edited(FULL, output_head__expansion_ref=None), "emptyField", "output_head.expansion_ref"),
    (edited(FULL, output_head__kind='"dense"'), "invalidOutputHead", "dense output head cannot declare factored weights or dimensions"),
    (edited(FULL, max_context="0"), "invalidMaxContext", 0),
    (edited(FULL, context_target_tokens="4096"), "invalidContextTarget", 4096),
    (edited(FULL, adapter_slots="-1"), "invalidAdapterSlots", -1),
    (edited(FULL, compression_policy__weight_bits="0"), "invalidWeightBits", 0),
    (edited(FULL, supported_backends="[]"), "missingBackends", None),
    (edited(FULL, supported_profiles="[]"), "missingProfiles", None),
    (edited(FULL, supported_backends='["metal"]'), "unsupportedValue", "metal"),
    (edited(FULL, model_tier='"turbo"'), "unsupportedValue", "turbo"),
    (edited(FULL, max_context='"2048"'), "unsupportedValue", "max_context"),
    (edited(FULL, format_version="1.1.0"), "unsupportedValue", "1.1.0"),
    (edited(FULL, signature_ref=None), "emptyField", "signature_ref"),
    (FULL.replace("[draft]", "[drafts]"), "malformedSection", "[drafts]"),
    (FULL + "just words\n", "malformedLine", "just words"),
])
def test_manifest_errors(text, case, payload):
    with pytest.raises(B.BundleError) as e:
        B.parse_manifest(text)
    assert e.value.case == case
    if isinstance(payload, str):
        assert e.value.text == payload
    elif payload is not None:
        assert e.value.detail == payload


def make_bundle(root, manifest=FULL, files=(("weights/cls_proj.bin", b"p"), ("weights/cls_expand.bin", b"e"), ("weights/future-sidecar.bin", b"{}"),
                                            ("weights/lm_head.bin", b"head"), ("tokenizer/tokenizer.model", b"tok"))):
    for entry in B.REQUIRED_TOP_LEVEL_ENTRIES:
        os.makedirs(os.path.join(root, entry), exist_ok=True)
    with open(os.path.join(root, "manifest.toml"), "w") as f:
        f.write(manifest)
    for rel, data in files:
        os.makedirs(os.path.dirname(os.path.join(root, rel)), exist_ok=True)
        with open(os.path.join(root, rel), "wb") as f:
            f.write(data)
    meta = {"name": "qwen3", "nLayer": 1, "nHead": 2, "nKVHead": 1, "dModel": 8, "headDim": 4, "hiddenDim": 16, "vocab": 32, "maxSeq": 16,
            "normEps": 1e-5, "ropeTheta": 10000.0, "eosToken": None, "architecture": "llama"}
    with open(os.path.join(root, "weights", "metadata.json"), "w") as f:
        json.dump(meta, f)


def hashlib_catalog(root):
    hashes = {}
    for d, _, names in os.walk(root):
        for n in names:
            rel = os.path.relpath(os.path.join(d, n), root).replace(os.sep, "/")
            if n == "manifest.toml" or rel == "signatures/content-hashes.json":
                continue
            hashes[rel] = hashlib.sha256(open(os.path.join(d, n), "rb").read()).hexdigest()
    return {"algorithm": "sha256", "manifestHash": hashlib.sha256(open(os.path.join(root, "manifest.toml"), "rb").read()).hexdigest(),
            "fileHashes": hashes}


# ---- ESPManifestTests.swift:448-496 (create/open round trip) with the catalog from either side ----
def test_bundle_opens_with_library_and_hashlib_catalogs(tmp_path):
    root = str(tmp_path / "model.esp")
    make_bundle(root)
    B.write_signature_catalog(root)
    written = json.load(open(os.path.join(root, "signatures", "content-hashes.json")))
    assert written == hashlib_catalog(root)                      # SHA-256 and the file enumeration agree with hashlib / os.walk
    b = B.RuntimeBundle(root)
    assert b.config.name == "qwen3" and b.config.d_model == 8
    json.dump(hashlib_catalog(root), open(os.path.join(root, "signatures", "content-hashes.json"), "w"))
    B.RuntimeBundle(root).close()
    # empty and multi-block inputs of the hash
    for size in (0, 1, 55, 56, 63, 64, 65, 119, 120, 1000):
        open(os.path.join(root, "weights", f"blob{size}.bin"), "wb").write(bytes(range(256)) * (size // 256) + bytes(range(size % 256)))
    B.write_signature_catalog(root)
    assert json.load(open(os.path.join(root, "signatures", "content-hashes.json"))) == hashlib_catalog(root)


# ---- :498-550 ----
def test_bundle_open_rejects_tampered_content(tmp_path):
    root = str(tmp_path / "model.esp")
    make_bundle(root)
    B.write_signature_catalog(root)
    open(os.path.join(root, "weights", "lm_head.bin"), "wb").write(b"tampered")
    with pytest.raises(B.BundleError) as e:
        B.RuntimeBundle(root)
    assert (e.value.case, e.value.text) == ("signatureMismatch", "weights/lm_head.bin")
    B.RuntimeBundle(root, verify_signatures=False).close()
    open(os.path.join(root, "weights", "lm_head.bin"), "wb").write(b"head")
    open(os.path.join(root, "manifest.toml"), "a").write("# touched\n")
    with pytest.raises(B.BundleError) as e:
        B.RuntimeBundle(root)
    assert (e.value.case, e.value.text) == ("signatureMismatch", "manifest.toml")


# ---- :380-446 and the layout checks of open (ESPBundle.swift:563-590, 641-692) ----
def test_bundle_open_checks_layout_and_references(tmp_path):
    root = str(tmp_path / "model.esp")
    make_bundle(root, files=(("weights/cls_proj.bin", b"p"), ("weights/cls_expand.bin", b"e")))
    B.write_signature_catalog(root)
    with pytest.raises(B.BundleError) as e:
        B.RuntimeBundle(root)
    assert (e.value.case, e.value.text) == ("missingReferencedFile", "weights/future-sidecar.bin")
    make_bundle(root, manifest=edited(FULL, draft__artifact_ref='"../outside.bin"'))
    with pytest.raises(B.BundleError) as e:
        B.RuntimeBundle(root, verify_signatures=False)
    assert (e.value.case, e.value.text) == ("invalidReferencedPath", "../outside.bin")
    make_bundle(root, manifest=edited(FULL, draft__artifact_ref='"/etc/passwd"'))
    with pytest.raises(B.BundleError) as e:
        B.RuntimeBundle(root, verify_signatures=False)
    assert e.value.case == "invalidReferencedPath"
    os.rmdir(os.path.join(root, "licenses"))
    with pytest.raises(B.BundleError) as e:
        B.RuntimeBundle(root, verify_signatures=False)
    assert (e.value.case, e.value.text) == ("missingTopLevelEntry", "licenses")
    os.remove(os.path.join(root, "manifest.toml"))
    with pytest.raises(B.BundleError) as e:
        B.RuntimeBundle(root, verify_signatures=False)
    assert e.value.case == "missingManifest"


# ---- ESPRuntimeResolverTests.swift:6-177, :179-265 ----
def test_backend_selection_and_environment_overrides(tmp_path):
    root = str(tmp_path / "model.esp")
    make_bundle(root)
    b = B.RuntimeBundle(root, verify_signatures=False)
    s = b.resolve()
    assert (s["backend"], s["profile"], s["context_target_tokens"], s["has_output_head"], s["has_draft"]) == ("ane-private", "prefill_2048", 1024, True, True)
    assert b.resolve(supports_ane_private=False)["backend"] == "cpu-safe"
    with pytest.raises(B.BundleError) as e:
        b.resolve(requested_context_tokens=1025)
    assert (e.value.case, e.value.detail, e.value.detail2) == ("requestedContextExceedsTarget", 1025, 1024)
    assert b.environment_overrides() == {
        "ESPRESSO_BUNDLE_OUTPUT_HEAD_KIND": "factored", "ESPRESSO_BUNDLE_OUTPUT_HEAD_BOTTLENECK": "128", "ESPRESSO_BUNDLE_OUTPUT_HEAD_GROUPS": "1",
        "ESPRESSO_BUNDLE_OUTPUT_HEAD_PROJECTION_REF": "weights/cls_proj.bin", "ESPRESSO_BUNDLE_OUTPUT_HEAD_EXPANSION_REF": "weights/cls_expand.bin",
        "ESPRESSO_BUNDLE_DRAFT_KIND": "exact_two_token", "ESPRESSO_BUNDLE_DRAFT_HORIZON": "2", "ESPRESSO_BUNDLE_DRAFT_VERIFIER": "exact",
        "ESPRESSO_BUNDLE_DRAFT_ROLLBACK": "exact_replay", "ESPRESSO_BUNDLE_DRAFT_ARTIFACT_REF": "weights/future-sidecar.bin",
        "ESPRESSO_BUNDLE_DRAFT_ACCEPTANCE_METRIC": "accepted_future_tokens"}
    b.close()
    # approximate heads and drafts are not passed on; a legacy bundle selects prefill_256
    make_bundle(root, manifest=edited(edited(FULL, draft__behavior_class='"approximate"'), output_head__behavior_class='"approximate"'))
    assert B.RuntimeBundle(root, verify_signatures=False).environment_overrides() == {}
    make_bundle(root, manifest=LEGACY)
    s = B.RuntimeBundle(root, verify_signatures=False).resolve(supports_ane_private=False)
    assert (s["backend"], s["profile"], s["reason"]) == ("cpu-safe", "prefill_256", "Fell back to CPU-safe backend")
    make_bundle(root, manifest=edited(LEGACY, supported_backends='["ane-private"]'))
    with pytest.raises(B.BundleError) as e:
        B.RuntimeBundle(root, verify_signatures=False).resolve(supports_ane_private=False)
    assert e.value.case == "noCompatibleBackend"
