"""Independent numpy restatements used to pin the C oracle.

Written from the published definitions (ggml block layouts, the llama decoder
equations), vectorised and in float64 where the C oracle is scalar float32, so
that a dropped term, wrong index or transposed operand in either shows up as a
disagreement.
"""
import numpy as np


# ---- GGUF blocks (public ggml layouts) ------------------------------------
def dequant_q8_0(blocks: np.ndarray) -> np.ndarray:
    b = blocks.reshape(-1, 34)
    d = b[:, :2].copy().view(np.float16).astype(np.float32)          # [nb,1]
    q = b[:, 2:].copy().view(np.int8).astype(np.float32)             # [nb,32]
    return (q * d).astype(np.float32).ravel()


def dequant_q4_0(blocks: np.ndarray) -> np.ndarray:
    b = blocks.reshape(-1, 18)
    d = b[:, :2].copy().view(np.float16).astype(np.float32)
    qs = b[:, 2:]
    lo = (qs & 0x0F).astype(np.int32) - 8
    hi = (qs >> 4).astype(np.int32) - 8
    vals = np.concatenate([lo, hi], axis=1).astype(np.float32)
    return (vals * d).astype(np.float32).ravel()


def q4_k_scales_mins(scales: np.ndarray):
    """scales: [nb,12] uint8 -> (sc [nb,8], m [nb,8]) 6-bit values."""
    s = scales.astype(np.uint16)
    sc = np.empty((s.shape[0], 8), dtype=np.uint16)
    m = np.empty((s.shape[0], 8), dtype=np.uint16)
    sc[:, :4] = s[:, 0:4] & 63
    m[:, :4] = s[:, 4:8] & 63
    sc[:, 4:] = (s[:, 8:12] & 0x0F) | ((s[:, 0:4] >> 6) << 4)
    m[:, 4:] = (s[:, 8:12] >> 4) | ((s[:, 4:8] >> 6) << 4)
    return sc, m


def dequant_q4_k(blocks: np.ndarray) -> np.ndarray:
    b = blocks.reshape(-1, 144)
    d = b[:, 0:2].copy().view(np.float16).astype(np.float32)         # [nb,1]
    dmin = b[:, 2:4].copy().view(np.float16).astype(np.float32)
    sc, m = q4_k_scales_mins(b[:, 4:16])
    d_eff = (d * sc.astype(np.float32)).astype(np.float32)           # fp32 product, rounded
    m_eff = (dmin * m.astype(np.float32)).astype(np.float32)
    qs = b[:, 16:].reshape(-1, 4, 32)                                # 4 chunks of 32 bytes
    nib = np.stack([qs & 0x0F, qs >> 4], axis=2).astype(np.float32)  # [nb,4,2,32] -> sub-block 2c+{0,1}
    nib = nib.reshape(-1, 8, 32)
    prod = (d_eff[:, :, None] * nib).astype(np.float32)
    return (prod - m_eff[:, :, None]).astype(np.float32).ravel()


# ---- decoder in float64 -----------------------------------------------------
def rmsnorm64(x, w, eps):
    x = x.astype(np.float64)
    return x / np.sqrt(np.mean(x * x) + eps) * w.astype(np.float64)


def rope64(v, heads, head_dim, pos, theta):
    v = v.astype(np.float64).reshape(heads, head_dim).copy()
    half = head_dim // 2
    i = np.arange(half, dtype=np.float64)
    ang = pos * theta ** (-2.0 * i / head_dim)
    c, s = np.cos(ang), np.sin(ang)
    a, b = v[:, :half].copy(), v[:, half:].copy()
    v[:, :half] = a * c - b * s
    v[:, half:] = a * s + b * c
    return v.ravel()


def silu64(x):
    return x / (1.0 + np.exp(-x))     # equals 0.5*x*(1+tanh(x/2)) analytically


class Llama64:
    """Plain float64 llama decoder with a token-major KV list (not channel-major)."""

    def __init__(self, cfg, weights):
        self.c, self.w = cfg, weights
        self.k = [[] for _ in range(cfg.n_layer)]
        self.v = [[] for _ in range(cfg.n_layer)]

    def forward(self, token):
        c, w = self.c, self.w
        pos = len(self.k[0])
        h = w["embedding"][token].astype(np.float64)
        group = c.n_head // c.n_kv_head
        for l in range(c.n_layer):
            L = w["layers"][l]
            a = rmsnorm64(h, L["rms_att"], c.norm_eps)
            q = rope64(L["wq"].astype(np.float64) @ a, c.n_head, c.head_dim, pos, c.rope_theta)
            k = rope64(L["wk"].astype(np.float64) @ a, c.n_kv_head, c.head_dim, pos, c.rope_theta)
            v = L["wv"].astype(np.float64) @ a
            self.k[l].append(k.reshape(c.n_kv_head, c.head_dim))
            self.v[l].append(v.reshape(c.n_kv_head, c.head_dim))
            K = np.stack(self.k[l])            # [t, kvh, hd]
            V = np.stack(self.v[l])
            ctx = np.empty((c.n_head, c.head_dim))
            for hh in range(c.n_head):
                kv = hh // group
                s = K[:, kv, :] @ q.reshape(c.n_head, c.head_dim)[hh] / np.sqrt(c.head_dim)
                p = np.exp(s - s.max())
                p /= p.sum()
                ctx[hh] = p @ V[:, kv, :]
            p_ = h + L["wo"].astype(np.float64) @ ctx.ravel()
            f = rmsnorm64(p_, L["rms_ffn"], c.norm_eps)
            g = L["w1"].astype(np.float64) @ f
            u = L["w3"].astype(np.float64) @ f
            h = p_ + L["w2"].astype(np.float64) @ (silu64(g) * u)
        return h

    def logits(self, h):
        return self.w["lm_head"].astype(np.float64) @ rmsnorm64(h, self.w["final_norm"], self.c.norm_eps)
