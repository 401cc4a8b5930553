"""Seeded synthetic llama weights shared by the oracle and GPU parity tests."""
import numpy as np

from oracle import oracle as orc

LAYER_SLOTS = {
    "rms_att": orc.W_RMS_ATT, "wq": orc.W_WQ, "wk": orc.W_WK, "wv": orc.W_WV, "wo": orc.W_WO,
    "rms_ffn": orc.W_RMS_FFN, "w1": orc.W_W1, "w2": orc.W_W2, "w3": orc.W_W3,
}
MATRICES = ("wq", "wk", "wv", "wo", "w1", "w2", "w3")


def matrix_shapes(cfg):
    ad, kd, d, hd = cfg.n_head * cfg.head_dim, cfg.n_kv_head * cfg.head_dim, cfg.d_model, cfg.hidden_dim
    return {"wq": (ad, d), "wk": (kd, d), "wv": (kd, d), "wo": (d, ad), "w1": (hd, d), "w3": (hd, d), "w2": (d, hd)}


def random_weights(cfg, seed, std=0.02, norm_jitter=0.0):
    """fp32 draws ~N(0,std) for every linear, embedding and head; norm weights 1 (+ optional jitter)."""
    rng = np.random.default_rng(seed)
    shapes = matrix_shapes(cfg)

    def norm_w(n):
        w = np.ones(n, dtype=np.float32)
        if norm_jitter:
            w += rng.normal(0, norm_jitter, n).astype(np.float32)
        return w

    w = {"embedding": rng.normal(0, std, (cfg.vocab, cfg.d_model)).astype(np.float32),
         "final_norm": norm_w(cfg.d_model),
         "lm_head": rng.normal(0, std, (cfg.vocab, cfg.d_model)).astype(np.float32),
         "layers": []}
    for _ in range(cfg.n_layer):
        L = {"rms_att": norm_w(cfg.d_model), "rms_ffn": norm_w(cfg.d_model)}
        for name in MATRICES:
            L[name] = rng.normal(0, std, shapes[name]).astype(np.float32)
        w["layers"].append(L)
    return w


def pack_weights(w, fmt, embedding_fmt=orc.FMT_F16):
    """Quantise every linear (and the head) to `fmt`; embedding and norms to fp16.
    Returns (packed, dequantised) where `dequantised` holds the fp32 values the packed bytes decode to."""
    packed = {"layers": []}
    deq = {"layers": []}

    def q(a, f):
        blocks = orc.quantize(f, a)
        return blocks, orc.dequantize(f, blocks, a.size).reshape(a.shape)

    packed["embedding"], deq["embedding"] = q(w["embedding"], embedding_fmt)
    packed["final_norm"], deq["final_norm"] = q(w["final_norm"], orc.FMT_F16)
    packed["lm_head"], deq["lm_head"] = q(w["lm_head"], fmt)
    for L in w["layers"]:
        P, D = {}, {}
        for name, a in L.items():
            P[name], D[name] = q(a, fmt if name in MATRICES else orc.FMT_F16)
        packed["layers"].append(P)
        deq["layers"].append(D)
    return packed, deq


def load_oracle(cfg, w):
    rt = orc.LlamaRuntime(cfg)
    rt.set_weight(0, orc.W_TOKEN_EMBEDDING, w["embedding"])
    rt.set_weight(0, orc.W_FINAL_NORM, w["final_norm"])
    rt.set_weight(0, orc.W_LM_HEAD, w["lm_head"])
    for l, L in enumerate(w["layers"]):
        for name, slot in LAYER_SLOTS.items():
            rt.set_weight(l, slot, L[name])
        if "q_norm" in L:
            rt.set_weight(l, orc.W_Q_NORM, L["q_norm"])
            rt.set_weight(l, orc.W_K_NORM, L["k_norm"])
    return rt
