"""A small GGUF (v3) writer for tests: typed metadata, tensor infos, aligned tensor data."""
import struct

import numpy as np

from oracle import oracle as orc

T_U32, T_I32, T_F32, T_BOOL, T_STRING, T_ARRAY, T_U64 = 4, 5, 6, 7, 8, 9, 10


def _s(x: str) -> bytes:
    b = x.encode()
    return struct.pack("<Q", len(b)) + b


def _value(v) -> bytes:
    if isinstance(v, bool):
        return struct.pack("<IB", T_BOOL, int(v))
    if isinstance(v, int):
        return struct.pack("<II", T_U32, v)
    if isinstance(v, float):
        return struct.pack("<If", T_F32, v)
    if isinstance(v, str):
        return struct.pack("<I", T_STRING) + _s(v)
    if isinstance(v, list):   # array of strings
        return struct.pack("<IIQ", T_ARRAY, T_STRING, len(v)) + b"".join(_s(x) for x in v)
    raise TypeError(type(v))


def write_gguf(path, metadata: dict, tensors: list, alignment: int = 32, version: int = 3):
    """tensors: [(name, ggml_type, (rows, cols) or (n,), raw_bytes[, offset written instead of the real one])]"""
    out = bytearray(struct.pack("<IIQQ", 0x46554747, version, len(tensors), len(metadata)))
    for k, v in metadata.items():
        out += _s(k) + _value(v)
    offset = 0
    for name, gtype, shape, raw, *forced_offset in tensors:
        dims = list(reversed(shape))                      # ne[0] is the innermost dimension
        out += _s(name) + struct.pack("<I", len(dims)) + b"".join(struct.pack("<Q", d) for d in dims)
        out += struct.pack("<IQ", gtype, forced_offset[0] if forced_offset else offset)
        offset += (len(raw) + alignment - 1) // alignment * alignment
    out += b"\0" * ((-len(out)) % alignment)
    for _, _, _, raw, *_ in tensors:
        out += bytes(raw) + b"\0" * ((-len(raw)) % alignment)
    open(path, "wb").write(bytes(out))


def gguf_model(path, kw, w, arch, matrix_fmt, tied=False, interleave_qk=True, mutate=None):
    """Writes a llama-family GGUF file the way llama.cpp's converter lays it out; returns the fp32 values
    (in the half-split row order the decoder uses) that the packed tensors decode to.  `mutate` may rewrite the tensor
    list (malformed files for the loader's error paths)."""
    hd, half = kw["head_dim"], kw["head_dim"] // 2

    def gguf_rows(a, heads):   # stored row (h, j, s) <- half-split row (h, s, j)
        if not interleave_qk:
            return a
        r = a.reshape(heads, 2, half, a.shape[1])
        return np.ascontiguousarray(r.transpose(0, 2, 1, 3)).reshape(a.shape)

    meta = {"general.architecture": arch, f"{arch}.block_count": kw["n_layer"], f"{arch}.attention.head_count": kw["n_head"],
            f"{arch}.attention.head_count_kv": kw["n_kv_head"], f"{arch}.embedding_length": kw["d_model"],
            f"{arch}.feed_forward_length": kw["hidden_dim"], f"{arch}.context_length": kw["max_seq"],
            f"{arch}.attention.layer_norm_rms_epsilon": 1e-5, f"{arch}.rope.freq_base": 10000.0,
            "tokenizer.ggml.tokens": [f"t{i}" for i in range(kw["vocab"])], "tokenizer.ggml.eos_token_id": 2,
            "general.name": "unit-test"}
    tensors, seen = [], {"layers": []}

    def quant(a):
        blocks = orc.quantize(matrix_fmt, a)
        return blocks, orc.dequantize(matrix_fmt, blocks, a.size).reshape(a.shape)

    emb16 = w["embedding"].astype(np.float16)
    tensors.append(("token_embd.weight", 1, w["embedding"].shape, emb16.tobytes()))
    seen["embedding"] = emb16.astype(np.float32)
    tensors.append(("output_norm.weight", 0, w["final_norm"].shape, w["final_norm"].astype("<f4").tobytes()))
    seen["final_norm"] = w["final_norm"]
    if tied:
        seen["lm_head"] = seen["embedding"]
    else:
        b, seen["lm_head"] = quant(w["lm_head"])
        tensors.append(("output.weight", matrix_fmt, w["lm_head"].shape, b.tobytes()))
    names = {"wq": "attn_q", "wk": "attn_k", "wv": "attn_v", "wo": "attn_output", "w1": "ffn_gate", "w2": "ffn_down", "w3": "ffn_up"}
    for l, L in enumerate(w["layers"]):
        S = {}
        for k, a in L.items():
            if k in names:
                b, S[k] = quant(a)
                stored = a
                if k == "wq": stored = gguf_rows(a, kw["n_head"])
                if k == "wk": stored = gguf_rows(a, kw["n_kv_head"])
                if stored is not a:
                    b = orc.quantize(matrix_fmt, stored)      # blocks lie within rows, so this is a row permutation of `b`
                tensors.append((f"blk.{l}.{names[k]}.weight", matrix_fmt, a.shape, b.tobytes()))
            else:
                g = {"rms_att": "attn_norm", "rms_ffn": "ffn_norm"}[k]
                tensors.append((f"blk.{l}.{g}.weight", 0, a.shape, a.astype("<f4").tobytes()))
                S[k] = a
        seen["layers"].append(S)
    write_gguf(path, meta, mutate(tensors) if mutate else tensors)
    return seen
