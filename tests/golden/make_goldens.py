"""Writes the golden fixtures of this directory from the CPU oracle (oracle/), which itself is pinned against the
reference's known-answer tests in tests/test_oracle_*.py.  Nothing from the reference is imported or run.

    python tests/golden/make_goldens.py

llama_decode.json   seeded tiny llama models (one per weight format and KV type): prompt, greedy tokens, logits of two steps,
                    the exact two-token stream with the reference loop's counters
blocks.json         packed GGUF blocks (Q8_0 / Q4_0 / Q4_K, random bytes with edge scales) and the fp32 bit patterns
                    they dequantise to
The models are rebuilt from the seeds by tests/model_util.py; the fixtures hold inputs that are not derivable from a
seed (block bytes) and every expected output.
"""
import base64
import json
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(HERE, ".."))
sys.path.insert(0, os.path.join(HERE, "..", ".."))

import model_util as mu  # noqa: E402
from oracle import oracle as orc  # noqa: E402

CONFIG = dict(n_layer=2, n_head=4, n_kv_head=2, d_model=256, head_dim=64, hidden_dim=512, vocab=512, max_seq=48)
FORMATS = {"q8_0": orc.FMT_Q8_0, "q4_0": orc.FMT_Q4_0, "q4_k": orc.FMT_Q4_K, "f16": orc.FMT_F16}
PROMPT = [3, 141, 59, 26, 5, 358, 97]


def build(fmt, seed, n_layer=None, kv_fp16=False):
    kw = dict(CONFIG, n_layer=n_layer or CONFIG["n_layer"])
    cfg = orc.LlamaConfig(gemv_inputs_fp16=True, kv_fp16=kv_fp16, **kw)
    w = mu.random_weights(cfg, seed, std=0.08, norm_jitter=0.05)
    packed, deq = mu.pack_weights(w, fmt)
    return kw, packed, mu.load_oracle(cfg, deq)


def llama_decode():
    cases = []
    for name, fmt in FORMATS.items():
        for kv_fp16 in (False, True):
            seed = 500 + fmt + (1 if kv_fp16 else 0)
            kw, _, rt = build(fmt, seed, kv_fp16=kv_fp16)
            rt.prefill(PROMPT)
            tokens, logits, margins = [], [], []
            for step in range(24):
                if step < 2:   # little-endian float32, base64
                    logits.append(base64.b64encode(np.asarray(rt.logits(), dtype="<f4").tobytes()).decode())
                margins.append(float(rt.top2_margin()))
                t = rt.select_greedy()
                tokens.append(int(t))
                rt.advance(t)
            case = {"format": name, "kv_fp16": kv_fp16, "seed": seed, "config": kw, "prompt": PROMPT, "tokens": tokens,
                    "logits_first_steps": logits, "min_top2_margin": min(margins)}
            if not kv_fp16:
                _, _, target = build(fmt, seed)
                _, _, draft = build(fmt, seed + 50, n_layer=1)
                stream, stats = orc.generate_two_token(target, draft, PROMPT, 24)
                case["two_token"] = {"draft_seed": seed + 50, "tokens": [int(t) for t in stream],
                                     "passes": int(stats["passes"]), "committed_total": int(stats["committed_total"]),
                                     "accepted_total": int(stats["accepted_total"])}
            cases.append(case)
    return {"about": "greedy decode of seeded tiny llama models on the CPU oracle (fp16 GEMV inputs, fp32 accumulation)", "cases": cases}


def blocks():
    rng = np.random.default_rng(2024)
    out = {"about": "GGUF blocks as hex and the uint32 bit patterns of their fp32 values", "cases": []}
    for name, fmt, block_bytes, elems in (("q8_0", orc.FMT_Q8_0, 34, 32), ("q4_0", orc.FMT_Q4_0, 18, 32), ("q4_k", orc.FMT_Q4_K, 144, 256)):
        n_blocks = 6
        raw = rng.integers(0, 256, n_blocks * block_bytes, dtype=np.uint8)
        # edge scales in the leading fp16 fields: zero, a subnormal, the largest finite value, negative
        for b, bits in enumerate((0x0000, 0x0001, 0x7BFF, 0xBC00, 0x3C00, 0x2E66)):
            raw[b * block_bytes: b * block_bytes + 2] = np.frombuffer(np.uint16(bits).tobytes(), np.uint8)
            if fmt == orc.FMT_Q4_K:   # dmin too
                raw[b * block_bytes + 2: b * block_bytes + 4] = np.frombuffer(np.uint16(bits ^ 0x8000).tobytes(), np.uint8)
        values = orc.dequantize(fmt, raw, n_blocks * elems)
        out["cases"].append({"format": name, "blocks_hex": raw.tobytes().hex(), "elements": n_blocks * elems,
                             "fp32_bits": [int(v) for v in values.view(np.uint32)]})
    return out


def main():
    for name, data in (("llama_decode.json", llama_decode()), ("blocks.json", blocks())):
        with open(os.path.join(HERE, name), "w") as f:
            json.dump(data, f, separators=(",", ":"))
            f.write("\n")
        print(name, os.path.getsize(os.path.join(HERE, name)), "bytes")


if __name__ == "__main__":
    main()
