"""Seeded random-init llama models in packed GGUF formats, built on the GPU (ops.synth_weights).

One stream id per tensor: stream = seed * 1000 + layer * 16 + tensor index, so a model is a pure
function of (config, seed, format)."""
from __future__ import annotations

import numpy as np

from . import _lib, llama, ops

_TENSORS = ("wq", "wk", "wv", "wo", "w1", "w2", "w3")


def matrix_shapes(cfg: llama.MultiModelConfig) -> dict:
    ad, kd, d, hd = cfg.attention_dim, cfg.kv_dim, cfg.d_model, cfg.hidden_dim
    return {"wq": (ad, d), "wk": (kd, d), "wv": (kd, d), "wo": (d, ad), "w1": (hd, d), "w3": (hd, d), "w2": (d, hd)}


def build_runtime(cfg: llama.MultiModelConfig, matrix_format: int, seed: int, std: float = 0.02,
                  kv_format: int = _lib.FORMAT_F32, max_sequences: int = 1, keep_packed: bool = False,
                  head_format: int | None = None, zero_upper_outputs: bool = False):
    """Random-init model: every linear ~N(0, std) in `matrix_format`, embedding fp16 ~N(0, std), norm weights 1.
    Returns (runtime, packed) where packed holds the GGUF-layout bytes when keep_packed is set.  Tensor seeds do not depend
    on the layer count, so a model built with fewer layers from the same seed is a prefix of the deeper one.
    zero_upper_outputs: wo and w2 of every layer above the first are all-zero blocks, i.e. those layers cost what they
    always cost and add nothing to the residual stream: the model's tokens are those of its first layer alone."""
    rt = llama.LlamaRuntime(cfg, kv_format=kv_format, max_sequences=max_sequences)
    shapes = matrix_shapes(cfg)
    head_format = matrix_format if head_format is None else head_format
    packed = {"layers": []} if keep_packed else None
    ones = np.ones(cfg.d_model, dtype=np.float16)

    def put(layer, name, slot, fmt, data):
        rt.set_weight(layer, slot, fmt, data)
        if packed is not None:
            (packed["layers"][layer] if layer >= 0 and name in llama.LAYER_SLOTS else packed)[name] = data

    base = seed * 1000
    emb = ops.synth_weights(_lib.FORMAT_F16, base + 1, std, cfg.vocab * cfg.d_model)
    put(-1, "embedding", llama.SLOT_TOKEN_EMBEDDING, _lib.FORMAT_F16, emb)
    put(-1, "final_norm", llama.SLOT_FINAL_NORM, _lib.FORMAT_F16, ones.view(np.uint8))
    head = ops.synth_weights(head_format, base + 2, std, cfg.vocab * cfg.d_model)
    put(-1, "lm_head", llama.SLOT_LM_HEAD, head_format, head)
    del emb, head
    for l in range(cfg.n_layer):
        if packed is not None:
            packed["layers"].append({})
        put(l, "rms_att", llama.SLOT_RMS_ATT, _lib.FORMAT_F16, ones.view(np.uint8))
        put(l, "rms_ffn", llama.SLOT_RMS_FFN, _lib.FORMAT_F16, ones.view(np.uint8))
        for i, name in enumerate(_TENSORS):
            r, c = shapes[name]
            if zero_upper_outputs and l >= 1 and name in ("wo", "w2"):
                data = np.zeros(ops.format_bytes(matrix_format, r * c), dtype=np.uint8)
            else:
                data = ops.synth_weights(matrix_format, base + 16 * (l + 1) + i, std, r * c)
            put(l, name, llama.LAYER_SLOTS[name], matrix_format, data)
    rt.finalize()
    return rt, packed


STORIES_6L = dict(n_layer=6, n_head=12, n_kv_head=12, d_model=768, head_dim=64, hidden_dim=2048, vocab=32000,
                  max_seq=256, norm_eps=1e-5, rope_theta=10000.0, name="stories-6l-d768")
LLAMA3_8B = dict(n_layer=32, n_head=32, n_kv_head=8, d_model=4096, head_dim=128, hidden_dim=14336, vocab=128256,
                 max_seq=1024, norm_eps=1e-5, rope_theta=500000.0, name="llama3-8b-arch")
